"""Mirror of the reference's `flex_gemm.kernels` package for the sparse-convolution path: `kernels.cuda` carries the
names of its pybind11 module (flex_gemm/kernels/cuda/ext.cpp:10-36), served by the gfx950 library."""
from . import cuda

__all__ = ["cuda"]
