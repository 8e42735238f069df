"""flexgemm_amd -- MI355X (gfx950) implementation of FlexGEMM's submanifold sparse-conv path.

`flexgemm_amd.ops.spconv` mirrors the reference's `flex_gemm.ops.spconv` interface; the `flex_gemm`
package next to this one re-exports it under the reference's import path.
"""
from . import kernels, ops  # noqa: F401
from .ops.spconv import (Algorithm, SubMConv3dFunction, SubMConv3dNeighborCache, set_algorithm,  # noqa: F401
                         set_hashmap_ratio, sparse_submanifold_conv3d)

__all__ = ["kernels", "ops", "Algorithm", "SubMConv3dFunction", "SubMConv3dNeighborCache", "set_algorithm",
           "set_hashmap_ratio", "sparse_submanifold_conv3d"]
