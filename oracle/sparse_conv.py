"""TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's generic sparse convolution
(stride / padding / dilation, output coordinates that differ from the input's).

Tables (numpy):
  * output_coords         -- flex_gemm/ops/spconv/sparse_conv3d.py:96-127 (torch builder) and
                             flex_gemm/kernels/cuda/spconv/sparse_neighbor_map.cu:19-57, 76-131 (native, BXYZ keys)
  * neighbor_maps         -- sparse_conv3d.py:224-278 (torch builder) and sparse_neighbor_map.cu:431-467 (native)
Arithmetic (torch, any float dtype; tests run it in float64):
  * forward / backward    -- sparse_conv3d.py:291-305 and :357-390 (explicit gather-GEMM)

Pinning (tests/test_oracle_sparse_conv.py): output coordinates and both maps against a brute-force
dictionary builder written from the definition; forward values and all three gradients against
torch.nn.functional.conv3d with the same stride / padding / dilation on small dense grids
(sampled at the output coordinates, gradients through autograd); with stride 1, padding K//2 and
out_coords = coords the maps reduce to the submanifold map and its column-flipped copy.
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import numpy as np
import torch

from .explicit_gemm import _as_index, _im2col

EMPTY = 0xFFFFFFFF


def out_dims(shape: Sequence[int], kernel_size, stride, padding, dilation) -> Tuple[int, int, int]:
    """(Wo, Ho, Do) = (W + 2P - D(K-1) - 1) // S + 1   (sparse_conv3d.py:105-107)."""
    _, _, W, H, D = [int(s) for s in shape]
    return tuple((n + 2 * p - d * (k - 1) - 1) // s + 1
                 for n, k, s, p, d in zip((W, H, D), kernel_size, stride, padding, dilation))


def kernel_offsets(kernel_size) -> np.ndarray:
    """[V, 3] kernel positions (kx, ky, kz), v = (kx*Kh + ky)*Kd + kz (sparse_neighbor_map.cu:40-42)."""
    kw, kh, kd = [int(k) for k in kernel_size]
    return np.stack(np.meshgrid(np.arange(kw), np.arange(kh), np.arange(kd), indexing="ij"), -1).reshape(-1, 3).astype(np.int64)


def output_coords(coords: np.ndarray, shape: Sequence[int], kernel_size, stride, padding, dilation) -> np.ndarray:
    """Sorted (b, x, y, z) list of every output cell that some input voxel reaches: o = (i + P - k*D) / S for a kernel
    position k, when the division is exact and o lies inside the output grid (sparse_conv3d.py:109-127)."""
    coords = np.asarray(coords, dtype=np.int64).reshape(-1, 4)
    dims = np.asarray(out_dims(shape, kernel_size, stride, padding, dilation), dtype=np.int64)
    k = kernel_offsets(kernel_size)
    s = np.asarray(stride, dtype=np.int64)
    p = np.asarray(padding, dtype=np.int64)
    d = np.asarray(dilation, dtype=np.int64)
    cand = coords[:, None, 1:] + p[None, None, :] - k[None, :, :] * d[None, None, :]          # [M, V, 3]
    batch = np.broadcast_to(coords[:, None, 0:1], cand.shape[:2] + (1,))
    ok = np.all(np.mod(cand, s) == 0, axis=-1)                   # python-style mod: a negative multiple still passes ...
    q = np.floor_divide(cand, s)
    ok &= np.all((q >= 0) & (q < dims), axis=-1)                 # ... and fails here
    rows = np.concatenate([batch, q], axis=-1)[ok]
    if rows.shape[0] == 0:
        return np.empty((0, 4), dtype=np.int32)
    return np.unique(rows, axis=0).astype(np.int32)


def neighbor_maps(coords: np.ndarray, out_coords: np.ndarray, shape: Sequence[int], kernel_size, stride, padding,
                  dilation, with_bwd: bool = True) -> Tuple[np.ndarray, Optional[np.ndarray]]:
    """fwd[o, v] = index of the input voxel at out_coords[o]*S - P + k_v*D (same batch, inside the grid), else all
    ones; bwd[i, v] = o for every fwd[o, v] = i (sparse_conv3d.py:243-272, sparse_neighbor_map.cu:448-466)."""
    coords = np.asarray(coords, dtype=np.int64).reshape(-1, 4)
    out_coords = np.asarray(out_coords, dtype=np.int64).reshape(-1, 4)
    _, _, W, H, D = [int(x) for x in shape]
    m, l = coords.shape[0], out_coords.shape[0]
    k = kernel_offsets(kernel_size)
    v = k.shape[0]
    s = np.asarray(stride, dtype=np.int64)
    p = np.asarray(padding, dtype=np.int64)
    d = np.asarray(dilation, dtype=np.int64)
    fwd = np.full((l, v), EMPTY, dtype=np.uint32)
    bwd = np.full((m, v), EMPTY, dtype=np.uint32) if with_bwd else None
    if m == 0 or l == 0:
        return fwd, bwd
    keys = ((coords[:, 0] * W + coords[:, 1]) * H + coords[:, 2]) * D + coords[:, 3]
    order = np.argsort(keys, kind="stable")
    skeys = keys[order]
    for j in range(v):
        q = out_coords[:, 1:] * s[None, :] - p[None, :] + k[j][None, :] * d[None, :]
        inside = (q[:, 0] >= 0) & (q[:, 0] < W) & (q[:, 1] >= 0) & (q[:, 1] < H) & (q[:, 2] >= 0) & (q[:, 2] < D)
        qk = ((out_coords[:, 0] * W + q[:, 0]) * H + q[:, 1]) * D + q[:, 2]
        pos = np.clip(np.searchsorted(skeys, qk), 0, m - 1)
        hit = inside & (skeys[pos] == qk)
        src = order[pos[hit]]
        fwd[hit, j] = src.astype(np.uint32)
        if with_bwd:
            bwd[src, j] = np.nonzero(hit)[0].astype(np.uint32)
    return fwd, bwd


def output_coords_bruteforce(coords, shape, kernel_size, stride, padding, dilation) -> np.ndarray:
    """Python sets on tuples, straight from the definition; small inputs only."""
    wo, ho, do = out_dims(shape, kernel_size, stride, padding, dilation)
    seen = set()
    for b, x, y, z in [tuple(int(t) for t in c) for c in coords]:
        for kx in range(kernel_size[0]):
            for ky in range(kernel_size[1]):
                for kz in range(kernel_size[2]):
                    o = (x + padding[0] - kx * dilation[0], y + padding[1] - ky * dilation[1], z + padding[2] - kz * dilation[2])
                    if any(c % st for c, st in zip(o, stride)):
                        continue
                    o = tuple(c // st for c, st in zip(o, stride))
                    if 0 <= o[0] < wo and 0 <= o[1] < ho and 0 <= o[2] < do:
                        seen.add((b,) + o)
    return np.asarray(sorted(seen), dtype=np.int32).reshape(-1, 4)


def neighbor_maps_bruteforce(coords, out_coords, shape, kernel_size, stride, padding, dilation):
    """Python dict on tuples; small inputs only."""
    _, _, W, H, D = [int(x) for x in shape]
    table = {tuple(int(t) for t in c): i for i, c in enumerate(coords)}
    kw, kh, kd = kernel_size
    v = kw * kh * kd
    fwd = np.full((len(out_coords), v), EMPTY, dtype=np.uint32)
    bwd = np.full((len(coords), v), EMPTY, dtype=np.uint32)
    for o, (b, x, y, z) in enumerate([tuple(int(t) for t in c) for c in out_coords]):
        for kx in range(kw):
            for ky in range(kh):
                for kz in range(kd):
                    j = (kx * kh + ky) * kd + kz
                    q = (x * stride[0] - padding[0] + kx * dilation[0], y * stride[1] - padding[1] + ky * dilation[1],
                         z * stride[2] - padding[2] + kz * dilation[2])
                    if not (0 <= q[0] < W and 0 <= q[1] < H and 0 <= q[2] < D):
                        continue
                    i = table.get((b,) + q)
                    if i is not None:
                        fwd[o, j] = i
                        bwd[i, j] = o
    return fwd, bwd


def forward(feats: torch.Tensor, neighbor_map, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[o] = bias + sum_v feats[fwd[o, v]] . W[:, v, :]^T   (sparse_conv3d.py:291-305)."""
    co, ci = weight.shape[0], weight.shape[-1]
    v = weight.numel() // (co * ci)
    idx = _as_index(torch.as_tensor(np.asarray(neighbor_map).astype(np.int64)) if isinstance(neighbor_map, np.ndarray) else neighbor_map)
    col = _im2col(feats, idx)
    w = weight.reshape(co, v * ci).t()
    return torch.addmm(bias, col, w) if bias is not None else torch.mm(col, w)


def backward(grad_output: torch.Tensor, feats: torch.Tensor, neighbor_map, neighbor_map_bwd, weight: torch.Tensor):
    """(grad_input [M, Ci], grad_weight [Co, Kw, Kh, Kd, Ci], grad_bias [Co])   (sparse_conv3d.py:357-390): the input
    gradient gathers grad_output through the backward map with the weight viewed [V*Co, Ci] (no flip of V)."""
    co, ci = weight.shape[0], weight.shape[-1]
    ksz = tuple(weight.shape[1:-1])
    v = weight.numel() // (co * ci)

    def as_idx(m):
        return _as_index(torch.as_tensor(np.asarray(m).astype(np.int64)) if isinstance(m, np.ndarray) else m)

    col = _im2col(grad_output, as_idx(neighbor_map_bwd))
    grad_input = torch.mm(col, weight.reshape(co, v, ci).transpose(0, 1).reshape(v * co, ci))
    col = _im2col(feats, as_idx(neighbor_map))
    grad_weight = torch.mm(col.t(), grad_output).view(v, ci, co).permute(2, 0, 1).contiguous().view(co, *ksz, ci)
    grad_bias = grad_output.sum(dim=0)
    return grad_input, grad_weight, grad_bias
