"""Drop-in import path: `import flex_gemm; from flex_gemm.ops.spconv import sparse_submanifold_conv3d`
resolves to the MI355X implementation in `flexgemm_amd` (same module objects, so `set_algorithm`
and the module-level `ALGORITHM` / `HASHMAP_RATIO` are shared)."""
import importlib
import sys

import flexgemm_amd as _impl

for _name in ("kernels", "kernels.cuda", "kernels.triton", "kernels.triton.spconv", "kernels.triton.spconv.config", "ops", "ops.utils", "ops.serialize", "ops.spconv", "ops.spconv.submanifold_conv3d", "ops.spconv.sparse_conv3d"):
    sys.modules[__name__ + "." + _name] = importlib.import_module("flexgemm_amd." + _name)

kernels = _impl.kernels
ops = _impl.ops
__all__ = ["kernels", "ops"]
