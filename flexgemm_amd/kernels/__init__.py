"""Mirror of the reference's `flex_gemm.kernels` package for the sparse-convolution path: `kernels.cuda` carries the
names of its pybind11 module (flex_gemm/kernels/cuda/ext.cpp:10-36), `kernels.triton` the kernel-level convolution calls
of its second package (flex_gemm/kernels/triton/spconv/__init__.py:1-13), both served by the gfx950 library."""
from . import cuda, triton

__all__ = ["cuda", "triton"]
