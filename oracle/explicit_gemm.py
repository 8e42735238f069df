"""TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's explicit gather-GEMM path.

Follows flex_gemm/ops/spconv/submanifold_conv3d.py:158-172 (forward) and :229-260 (backward):
a zero-filled im2col buffer [rows * V, C] receives the gathered neighbor rows, is viewed as
[rows, V * C] and multiplied with the flattened weight.  The only departure is row chunking,
which bounds the im2col buffer (the full buffer is N * 27 * C elements) without changing any
product: every output row depends on its own im2col row only, and the weight gradient is a sum
over rows, accumulated across chunks in the compute dtype.

Pinning (tests/test_oracle_gemm.py): dense torch.nn.functional.conv3d on small grids (values
and autograd gradients), the single-voxel closed form, the all-ones-weight neighbor sum,
linearity, and chunk-size invariance.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

EMPTY = 0xFFFFFFFF


def _as_index(neighbor_map: torch.Tensor) -> torch.Tensor:
    """uint32/int32/int64 map -> int64 with -1 for absent neighbors."""
    if neighbor_map.dtype == torch.uint32:
        neighbor_map = neighbor_map.view(torch.int32)
    m = neighbor_map.to(torch.int64)
    return torch.where((m == EMPTY) | (m < 0), torch.full_like(m, -1), m)


def _im2col(src: torch.Tensor, idx: torch.Tensor) -> torch.Tensor:
    """src [N, C], idx [R, V] (-1 = absent) -> [R, V*C] with zero rows for absent neighbors."""
    r, v = idx.shape
    c = src.shape[1]
    buf = torch.zeros((r * v, c), dtype=src.dtype)
    flat = idx.reshape(-1)
    mask = flat >= 0
    buf[mask] = src[flat[mask]]
    return buf.view(r, v * c)


def forward(feats: torch.Tensor, neighbor_map: torch.Tensor, weight: torch.Tensor,
            bias: Optional[torch.Tensor] = None, chunk_rows: int = 65536) -> torch.Tensor:
    """out = addmm(bias, im2col, W.view(Co, V*Ci).T)   (submanifold_conv3d.py:161-172)."""
    co = weight.shape[0]
    ci = weight.shape[-1]
    v = weight.numel() // (co * ci)
    idx = _as_index(neighbor_map)
    n = idx.shape[0]
    w = weight.reshape(co, v * ci).t()
    out = torch.empty((n, co), dtype=feats.dtype)
    for s in range(0, n, chunk_rows):
        col = _im2col(feats, idx[s:s + chunk_rows])
        out[s:s + chunk_rows] = torch.addmm(bias, col, w) if bias is not None else torch.mm(col, w)
    return out


def backward(grad_output: torch.Tensor, feats: torch.Tensor, neighbor_map: torch.Tensor, weight: torch.Tensor,
             need_input: bool = True, need_weight: bool = True, need_bias: bool = True,
             chunk_rows: int = 65536) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor]]:
    """(grad_input, grad_weight, grad_bias)   (submanifold_conv3d.py:229-260)."""
    co = weight.shape[0]
    ci = weight.shape[-1]
    ksz = tuple(weight.shape[1:-1])
    v = weight.numel() // (co * ci)
    idx = _as_index(neighbor_map)
    n = idx.shape[0]
    grad_input = grad_weight = grad_bias = None
    if need_input:
        # :233-241 -- gather grad_output through the map flipped along V, weight viewed [V*Co, Ci]
        inv = torch.flip(idx, [1])
        wt = weight.reshape(co, v, ci).transpose(0, 1).reshape(v * co, ci)
        grad_input = torch.empty((n, ci), dtype=grad_output.dtype)
        for s in range(0, n, chunk_rows):
            grad_input[s:s + chunk_rows] = torch.mm(_im2col(grad_output, inv[s:s + chunk_rows]), wt)
    if need_weight:
        # :246-253 -- im2col.T @ grad_output -> [V*Ci, Co] -> [Co, V, Ci]
        acc = torch.zeros((v * ci, co), dtype=feats.dtype)
        for s in range(0, n, chunk_rows):
            acc += torch.mm(_im2col(feats, idx[s:s + chunk_rows]).t(), grad_output[s:s + chunk_rows])
        grad_weight = acc.view(v, ci, co).permute(2, 0, 1).contiguous().view(co, *ksz, ci)
    if need_bias:
        grad_bias = grad_output.sum(dim=0)   # :257-258
    return grad_input, grad_weight, grad_bias


def weight_grad_offset(grad_output: torch.Tensor, feats: torch.Tensor, neighbor_map: torch.Tensor, v: int,
                       chunk_rows: int = 262144) -> torch.Tensor:
    """grad_weight[:, v, :] alone, [Co, Ci]: column v of the im2col product of submanifold_conv3d.py:246-253, i.e. the
    sum over the rows n with a neighbor at offset v of grad_output[n]^T feats[neighbor_map[n, v]].  For full-size
    workloads, where the whole [V*Ci, Co] product is too slow; tests/test_oracle_gemm.py pins it to backward()."""
    idx = _as_index(neighbor_map)[:, v]
    rows = torch.nonzero(idx >= 0).reshape(-1)
    acc = torch.zeros((grad_output.shape[1], feats.shape[1]), dtype=feats.dtype)
    for s in range(0, rows.numel(), chunk_rows):
        r = rows[s:s + chunk_rows]
        acc += torch.mm(grad_output[r].t(), feats[idx[r]])
    return acc


def calc_err(src: torch.Tensor, ref: torch.Tensor) -> Tuple[float, float]:
    """max / mean over elements of min(abs err, rel err), rel clamp 1e-6 (reference tests/utils.py:28-32)."""
    abs_err = (src.double() - ref.double()).abs()
    rel_err = abs_err / ref.double().abs().clamp_min(1e-6)
    err = torch.minimum(abs_err, rel_err)
    return float(err.max()), float(err.mean())


def max_rel_err(src: torch.Tensor, ref: torch.Tensor) -> float:
    """Maximum error relative to the reference tensor's scale: max|src-ref| / max|ref|."""
    denom = float(ref.double().abs().max())
    return float((src.double() - ref.double()).abs().max()) / max(denom, 1e-30)
