"""Synthetic workloads for the submanifold-conv hot path (host side, numpy + torch CPU).

The five benchmark configurations are thin spherical voxel shells: a voxel with integer
index (x, y, z) in [0, res)^3 is active iff the distance of its centre (idx + 0.5) to the
grid centre (res/2, res/2, res/2) lies within 0.5 of the radius 0.45 * res.  Voxels are
enumerated x-major, then y, then z (the same order `numpy.nonzero` of a dense predicate
would give); configuration 4 additionally shuffles the rows with a seeded permutation.

The reference's own test geometry (tests/utils.py:6-25, a thicker shell hugging the grid
boundary) is provided as `reference_test_shell` because the reference's neighbor-map
test (tests/submconv/neighbor_cache.py:63-93) sweeps it over res = 1 ... 512.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

import numpy as np
import torch

__all__ = [
    "shell_coords", "reference_test_shell", "ConvWorkload", "CONFIGS", "make_workload",
    "valid_pairs",
]


def _shell_from_bounds(res: int, lo4: int, hi4: int) -> np.ndarray:
    """All (x, y, z) in [0,res)^3 with lo4 <= (2x+1-res)^2+(2y+1-res)^2+(2z+1-res)^2 <= hi4.

    Integer arithmetic on 4*d^2 keeps the predicate exact.  O(res^2 + N): for every (x, y)
    column the admissible |2z+1-res| interval is bracketed with a float sqrt, widened by one
    and filtered with the exact integer test.
    """
    if res <= 0 or hi4 < lo4:
        return np.zeros((0, 3), dtype=np.int32)
    w = 2 * np.arange(res, dtype=np.int64) + 1 - res          # odd/even ints, ascending
    s_xy = (w[:, None] ** 2 + w[None, :] ** 2).reshape(-1)     # [res*res], x-major
    rem_hi = hi4 - s_xy
    keep = rem_hi >= 0
    col = np.nonzero(keep)[0]
    if col.size == 0:
        return np.zeros((0, 3), dtype=np.int32)
    s_xy = s_xy[col]
    rem_hi = rem_hi[col]
    rem_lo = np.maximum(lo4 - s_xy, 0)
    wmax = np.floor(np.sqrt(rem_hi.astype(np.float64))).astype(np.int64) + 1
    wmin = np.maximum(np.ceil(np.sqrt(rem_lo.astype(np.float64))).astype(np.int64) - 1, 0)
    # Two candidate z intervals per column (w_z < 0 side, then w_z > 0 side), each widened
    # by the +-1 slack above and filtered with the exact predicate afterwards.
    a_lo = np.maximum((res - 1 - wmax) // 2, 0)
    a_hi = np.minimum((res - 1 - wmin) // 2 + 1, res - 1)
    b_lo = np.maximum(np.maximum((res - 1 + wmin) // 2, 0), a_hi + 1)
    b_hi = np.minimum((res - 1 + wmax) // 2 + 1, res - 1)
    lo2 = np.stack([a_lo, b_lo], axis=1).reshape(-1)           # interval-major inside a column
    hi2 = np.stack([a_hi, b_hi], axis=1).reshape(-1)
    cnt = np.maximum(hi2 - lo2 + 1, 0)
    total = int(cnt.sum())
    if total == 0:
        return np.zeros((0, 3), dtype=np.int32)
    start = np.cumsum(cnt) - cnt
    owner = np.repeat(np.arange(col.size * 2), cnt) // 2
    z = np.arange(total, dtype=np.int64) - np.repeat(start, cnt) + np.repeat(lo2, cnt)
    wz2 = (2 * z + 1 - res) ** 2
    s = s_xy[owner] + wz2
    ok = (s >= lo4) & (s <= hi4)
    owner = owner[ok]
    z = z[ok]
    xy = col[owner]
    out = np.stack([xy // res, xy % res, z], axis=1).astype(np.int32)
    return out


def shell_coords(res: int, radius_frac: float = 0.45, half_thickness: float = 0.5,
                 batch: int = 1) -> np.ndarray:
    """int32 [N, 4] rows (b, x, y, z) of the benchmark shell at resolution `res`."""
    r = radius_frac * res
    lo = max(r - half_thickness, 0.0)
    hi = r + half_thickness
    lo4 = int(math.ceil(4.0 * lo * lo))
    hi4 = int(math.floor(4.0 * hi * hi))
    xyz = _shell_from_bounds(res, lo4, hi4)
    return _with_batch(xyz, batch)


def reference_test_shell(res: int, batch: int = 1) -> np.ndarray:
    """The reference's test geometry: res/2 - 1.25 <= |idx - res/2 + 0.5| <= res/2.

    Restates tests/utils.py:6-25 (chunking by 256^3 there only bounds memory; the chunks
    are concatenated chunk-major, so for res <= 256 the order is plain x-major and for
    larger res this function's x-major order is a permutation of the reference's).
    """
    hi = res / 2.0
    lo = max(res / 2.0 - 1.25, 0.0)
    # |idx + 0.5 - res/2| is the same half-integer lattice as the benchmark shell
    lo4 = int(math.ceil(4.0 * lo * lo))
    hi4 = int(math.floor(4.0 * hi * hi))
    xyz = _shell_from_bounds(res, lo4, hi4)
    return _with_batch(xyz, batch)


def _with_batch(xyz: np.ndarray, batch: int) -> np.ndarray:
    n = xyz.shape[0]
    out = np.empty((n * batch, 4), dtype=np.int32)
    for b in range(batch):
        out[b * n:(b + 1) * n, 0] = b
        out[b * n:(b + 1) * n, 1:] = xyz
    return out


@dataclass
class ConvWorkload:
    """One benchmark configuration, fully materialised on the CPU."""
    name: str
    res: int
    channels: int
    dtype: torch.dtype
    coords: torch.Tensor           # int32 [N, 4]
    shape: torch.Size              # (B, C, W, H, D)
    feats: torch.Tensor            # [N, Ci]  fp32 master copy
    weight: torch.Tensor           # [Co, 3, 3, 3, Ci] fp32 master copy
    bias: torch.Tensor             # [Co] fp32 master copy
    grad: torch.Tensor             # [N, Co] fp32 master copy (upstream gradient)

    @property
    def n(self) -> int:
        return int(self.coords.shape[0])


# name -> (res, C, dtype, shuffle, seed)
CONFIGS = {
    "cfg1": (64, 64, torch.float32, False, 1),
    "cfg2": (256, 256, torch.float16, False, 2),
    "cfg3": (512, 128, torch.float16, False, 3),
    "cfg4": (1024, 32, torch.bfloat16, True, 4),
    "cfg5": (128, 1024, torch.float16, False, 5),
}


def make_workload(name: str, res: Optional[int] = None, channels: Optional[int] = None,
                  dtype: Optional[torch.dtype] = None, with_values: bool = True) -> ConvWorkload:
    """Build configuration `name` (optionally overriding res / channels / dtype for scaled-down tests).

    Values come from a seeded CPU generator in fp32: feats ~ N(0,1), weight ~ N(0,1)/sqrt(27*Ci),
    bias ~ N(0,1), upstream grad ~ N(0,1).  Callers cast to the working dtype.
    """
    r0, c0, d0, shuffle, seed = CONFIGS[name]
    res = r0 if res is None else res
    c = c0 if channels is None else channels
    dt = d0 if dtype is None else dtype
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    coords = torch.from_numpy(shell_coords(res))
    if shuffle:
        coords = coords[torch.randperm(coords.shape[0], generator=g)].contiguous()
    n = coords.shape[0]
    if with_values:
        feats = torch.randn(n, c, generator=g)
        weight = torch.randn(c, 3, 3, 3, c, generator=g) / math.sqrt(27 * c)
        bias = torch.randn(c, generator=g)
        grad = torch.randn(n, c, generator=g)
    else:
        feats = weight = bias = grad = torch.empty(0)
    return ConvWorkload(name, res, c, dt, coords, torch.Size([1, c, res, res, res]),
                        feats, weight, bias, grad)


def valid_pairs(neighbor_map: torch.Tensor) -> int:
    """L = number of (voxel, offset) pairs with a present neighbor (reference tests/submconv/fwd.py:247)."""
    if neighbor_map.dtype == torch.uint32:
        neighbor_map = neighbor_map.view(torch.int32)
    return int((neighbor_map != -1).sum().item())
