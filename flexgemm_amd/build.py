"""Build recipe of libflexgemm_hip.so: hipcc, gfx950 only, in-tree output.

`python -m flexgemm_amd.build` compiles every file under flexgemm_amd/csrc/ and links
flexgemm_amd/_lib/libflexgemm_hip.so, then the tests' torch-free caller of the C ABI against it
(flexgemm_amd/_lib/conv_host).  Objects are rebuilt when their source (or a header) is newer; pass
--force to rebuild everything.
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
OUT_DIR = os.path.join(PKG, "_lib")
LIB = os.path.join(OUT_DIR, "libflexgemm_hip.so")
# a caller of the C ABI without Python or torch, run by the GPU tests (tests/cabi_host/conv_host.cpp)
HOST_CHECK_SRC = os.path.join(PKG, "..", "tests", "cabi_host", "conv_host.cpp")
HOST_CHECK = os.path.join(OUT_DIR, "conv_host")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

COMMON_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
    "-DNDEBUG",
]


def _headers():
    return glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(PKG, "..", "include", "*.h"))


def _stale(target: str, deps) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force: bool = False, verbose: bool = True, jobs: int = 4) -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not sources:
        raise RuntimeError("no HIP sources found under " + CSRC)
    hdrs = _headers()
    objs = []
    todo = []
    for src in sources:
        obj = os.path.join(OUT_DIR, os.path.basename(src)[:-4] + ".o")
        objs.append(obj)
        if force or _stale(obj, [src] + hdrs):
            todo.append((src, obj))

    def compile_one(item):
        src, obj = item
        cmd = [HIPCC] + COMMON_FLAGS + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
        warn = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if verbose and warn:
            print(warn, flush=True)

    with ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        list(ex.map(compile_one, todo))
    if force or todo or _stale(LIB, objs):
        cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-fno-gpu-rdc"] + objs + ["-o", LIB]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if os.path.exists(HOST_CHECK_SRC) and (force or todo or _stale(HOST_CHECK, [HOST_CHECK_SRC, LIB] + hdrs)):
        cmd = [HIPCC] + COMMON_FLAGS + ["-I", os.path.join(PKG, "..", "include"), HOST_CHECK_SRC, "-L", OUT_DIR, "-lflexgemm_hip",
                                        "-Wl,-rpath,$ORIGIN", "-o", HOST_CHECK]
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"building the host check failed:\n{r.stdout}\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
