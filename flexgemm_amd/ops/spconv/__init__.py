"""Algorithm switch and defaults of the sparse-conv operators
(same names and semantics as flex_gemm/ops/spconv/__init__.py:1-37)."""


class Algorithm:
    """Algorithm choices for sparse convolution.

    On gfx950 the four implicit-GEMM values share the same gather-GEMM kernels.  MASKED_* walk the
    mask-sorted row order and skip, tile by tile, the offsets no row of the tile has; IMPLICIT_GEMM*
    walk the rows in their natural order and every tile visits all offsets (for inputs so dense that
    sorting buys nothing), and their neighbor cache is the map alone.  The values without _SPLITK never
    split K.  EXPLICIT_GEMM is the gather + dense-GEMM formulation in torch ops."""
    EXPLICIT_GEMM = "explicit_gemm"
    IMPLICIT_GEMM = "implicit_gemm"
    IMPLICIT_GEMM_SPLITK = "implicit_gemm_splitk"
    MASKED_IMPLICIT_GEMM = "masked_implicit_gemm"
    MASKED_IMPLICIT_GEMM_SPLITK = "masked_implicit_gemm_splitk"


ALGORITHM = Algorithm.MASKED_IMPLICIT_GEMM_SPLITK  # Default algorithm
HASHMAP_RATIO = 2.0                                 # Ratio of hashmap size to input size


def set_algorithm(algorithm: str):
    global ALGORITHM
    ALGORITHM = algorithm


def set_hashmap_ratio(ratio: float):
    global HASHMAP_RATIO
    HASHMAP_RATIO = ratio


from .submanifold_conv3d import SubMConv3dFunction, SubMConv3dNeighborCache, sparse_submanifold_conv3d  # noqa: E402
