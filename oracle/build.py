"""Build recipe for the C oracle (TEST INFRASTRUCTURE ONLY).

`python -m oracle.build` compiles oracle/subm_ref.c into oracle/libsubm_ref.so with gcc.
The reference's own native code for this path (flex_gemm/kernels/cuda/**) is a torch C++/CUDA
extension: it needs torch/extension.h, device code compilation and a GPU to run, so no
oracle/_ref build of it exists here.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "subm_ref.c")
LIB = os.path.join(HERE, "libsubm_ref.so")


def build(force: bool = True) -> str:
    if not force and os.path.exists(LIB) and os.path.getmtime(LIB) >= os.path.getmtime(SRC):
        return LIB
    cmd = ["gcc", "-O2", "-std=c11", "-Wall", "-Wextra", "-shared", "-fPIC", SRC, "-o", LIB]
    subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    print(build(force=True))
    sys.exit(0)
