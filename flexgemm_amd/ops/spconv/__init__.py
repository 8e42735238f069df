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


class SerializationMode:
    """How 3-D coordinates are flattened into the key that orders generated output coordinates
    (flex_gemm/ops/spconv/__init__.py:10-14): by flattened (b, x, y, z) key, along the z-order curve or along the Hilbert
    curve."""
    BXYZ = 0
    Z_ORDER = 1
    HILBERT = 2


class SparseConv3dOutCoordAlgorithm:
    """Algorithm choices for generating output coordinates (flex_gemm/ops/spconv/__init__.py:17-20).  Both values give
    the same sorted list; on gfx950 they share one streaming implementation (candidate keys, radix sort, unique)."""
    HASHMAP = 0
    EXPAND_UNIQUE = 1


ALGORITHM = Algorithm.MASKED_IMPLICIT_GEMM_SPLITK  # Default algorithm
HASHMAP_RATIO = 2.0                                 # Ratio of hashmap size to input size
OUT_COORD_HASHMAP_RATIO = 1.1                       # kept for interface parity; the sort-based builder has no table
OUT_COORD_ALGO = SparseConv3dOutCoordAlgorithm.HASHMAP
SERIALIZATION_MODE = SerializationMode.BXYZ


# How the submanifold neighbor map is found (no counterpart in the reference, which always hashes; the map is the same
# either way): "hash" = open-addressing table and probes, "sort" = radix sort of the flattened keys and windowed merges,
# "auto" = "sort" once the searches outweigh the two sorts: from SORT_BUILDER_MIN_PROBES (voxel, kernel position)
# questions on (131 072 voxels of a 3x3x3 kernel).
NEIGHBOR_MAP_BUILDER = "auto"
SORT_BUILDER_MIN_PROBES = 27 * 131072
# How the streaming GEMM's tiles are dealt to its persistent workgroups: "balanced" (by cost, every round of tiles dealt
# expensive-first to the least loaded workgroup), "default" (the kernel's own round-robin over the tile list) or "auto"
# (balanced, except for the locality order of short-row layers, whose neighboring tiles are meant to share an XCD).
# The result does not depend on it.
GEMM_ITEM_ORDER = "auto"
# Narrow layers (16-bit, 8 ... 32 channels on both sides, submanifold): the gather GEMM that keeps a chunk's source rows
# resident in LDS (fgx_conv_narrow_gemm; 0.32 -> 0.19 ms per pass at 2.67 M voxels x 32 channels).  "auto": from 32 768
# rows on, once a neighbor cache has served three such products on the streaming kernel (sixteen below half a million
# rows: the plan it needs costs half of building the cache; a cache made for training with half a million voxels and more gets it at its second product,
# because the weight gradients gain the most); "on": whenever it fits; "off": never.
NARROW_RESIDENT = "auto"
# The bias gradient of a submanifold layer comes out of the streaming wgrad kernel (which loads every grad_output row for
# the centre offset anyway) instead of a column-sum pass of its own.  False: always the separate pass.
FUSE_DBIAS = True
# The fused-ReLU forward (sparse_submanifold_conv3d_relu) leaves the activation's derivative as one bit per output and
# backward masks the gradient with it (fgx_relu_mask_apply).  False: backward tests the saved output instead
# (torch.where), which reads the output again.
RELU_BIT_MASK = True


# Keep the repacked weight panels of the gather GEMMs with the weight tensor and reuse them while the weight is unchanged
# (no counterpart in the reference, whose kernels read the weight as it lies).  For serving and for gradient
# accumulation: a panel is kept from the second time a weight is seen at the same version counter and data pointer, so a
# loop that updates its weights every step keeps nothing.  Off by default, because the check cannot see a weight changed
# through `weight.data` (that path does not move the version counter): switch it on only where weights are updated
# through the tensor itself (torch.optim does) or not at all.  WEIGHT_PANEL_CACHE_MAX_BYTES bounds what is kept per
# process; beyond it panels are packed per call as without the cache.
WEIGHT_PANEL_CACHE = False
WEIGHT_PANEL_CACHE_MAX_BYTES = 4 << 30


def set_weight_panel_cache(enabled: bool, max_bytes: int = None):
    global WEIGHT_PANEL_CACHE, WEIGHT_PANEL_CACHE_MAX_BYTES
    WEIGHT_PANEL_CACHE = bool(enabled)
    if max_bytes is not None:
        WEIGHT_PANEL_CACHE_MAX_BYTES = int(max_bytes)


def set_neighbor_map_builder(builder: str):
    global NEIGHBOR_MAP_BUILDER
    if builder not in ("auto", "hash", "sort"):
        raise ValueError(f"unknown neighbor map builder {builder!r}; expected 'auto', 'hash' or 'sort'")
    NEIGHBOR_MAP_BUILDER = builder


def set_algorithm(algorithm: str):
    global ALGORITHM
    ALGORITHM = algorithm


def set_hashmap_ratio(ratio: float):
    global HASHMAP_RATIO
    HASHMAP_RATIO = ratio


from .submanifold_conv3d import (SubMConv3dFunction, SubMConv3dNeighborCache, sparse_submanifold_conv3d,  # noqa: E402
                                 sparse_submanifold_conv3d_relu)
from .sparse_conv3d import SparseConv3dFunction, SparseConv3dNeighborCache, sparse_conv3d, sparse_conv3d_relu  # noqa: E402
