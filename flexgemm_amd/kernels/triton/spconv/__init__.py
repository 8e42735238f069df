"""Kernel-level entry points of the implicit-GEMM convolutions, with the names, argument orders and return values of
the reference's package (flex_gemm/kernels/triton/spconv/__init__.py:1-13): tensors in, tensors out, no neighbor-cache
object.  Weights are [Co, V, Ci]; a backward call returns (grad_input, grad_weight [Co, V, Ci], grad_bias), each None
when its tensor does not require a gradient (..._bwd_implicit_gemm.py:177-225).

Each call runs the gfx950 gather-GEMM / wgrad kernels through the same host code as the operators.  The tables those
kernels walk (tile masks, gather plans, wgrad block bounds) are derived once from the `neighbor` tensor handed in and
kept on that tensor object, so calling again with the same map costs nothing extra; a map modified in place must be
passed as a new tensor.  `valid_kernel` / `valid_kernel_seg` callbacks are accepted and not called: the kernels' tile
sizes come from the fixed schedule table and their per-tile offset masks from `sorted_idx` and the map itself.  SPLITK,
which the reference's autotuner fills in, is accepted and ignored for the same reason.
"""
from __future__ import annotations

import ctypes as C
from typing import Callable, Optional, Tuple

import torch

from .... import _native as nat
from ....ops.spconv.submanifold_conv3d import SubMConv3dNeighborCache, _colsum, _gather_gemm, _require_cuda, _wgrad
from . import config

__all__ = [
    "sparse_submanifold_conv_fwd_implicit_gemm", "sparse_submanifold_conv_bwd_implicit_gemm",
    "sparse_submanifold_conv_fwd_implicit_gemm_splitk", "sparse_submanifold_conv_bwd_implicit_gemm_splitk",
    "sparse_submanifold_conv_fwd_masked_implicit_gemm", "sparse_submanifold_conv_bwd_masked_implicit_gemm",
    "sparse_submanifold_conv_fwd_masked_implicit_gemm_splitk", "sparse_submanifold_conv_bwd_masked_implicit_gemm_splitk",
    "sparse_conv_fwd_implicit_gemm", "sparse_conv_bwd_implicit_gemm",
    "sparse_conv_fwd_implicit_gemm_splitk", "sparse_conv_bwd_implicit_gemm_splitk",
    "sparse_conv_fwd_masked_implicit_gemm", "sparse_conv_bwd_masked_implicit_gemm",
    "sparse_conv_fwd_masked_implicit_gemm_splitk", "sparse_conv_bwd_masked_implicit_gemm_splitk",
    "config",
]

_GIVEN = ("sorted_idx", "valid_signal_i", "valid_signal_o", "valid_signal_seg")


def _fits(tables: SubMConv3dNeighborCache, given: dict) -> bool:
    for k, v in given.items():
        mine = getattr(tables, "_given_" + k, None)
        if mine is not None:
            if mine is not v:
                return False
        elif hasattr(tables, k):        # derived from the map in the meantime: not the caller's list
            return False
    return True


def _tables_of(neighbor: torch.Tensor, **given) -> SubMConv3dNeighborCache:
    """The derived tables that belong to `neighbor` and to the caller's own lists in `given` (matched by identity;
    the last four combinations seen with this map are kept)."""
    _require_cuda(neighbor, "flex_gemm.kernels.triton")
    assert neighbor.is_contiguous(), "Matrix neighbor must be contiguous"
    assert neighbor.dtype == torch.uint32 and neighbor.ndim == 2 and neighbor.shape[1] <= 32, "neighbor must be uint32 [N, V <= 32]"
    given = {k: v for k, v in given.items() if v is not None}
    n, v = neighbor.shape
    for k, t in given.items():
        assert t.is_cuda and t.device == neighbor.device, f"{k} must live on the device of neighbor"
        if k == "sorted_idx":
            assert t.dtype == torch.int64 and tuple(t.shape) == (n,), "sorted_idx must be int64 [N]"
        else:
            assert t.dtype == torch.uint32 and t.ndim == 1, f"{k} must be a uint32 vector"
    if "valid_signal_seg" in given:
        assert given["valid_signal_seg"].shape[0] == v + 1, "valid_signal_seg must have V + 1 entries"
    if "valid_signal_i" in given and "valid_signal_o" in given:
        assert given["valid_signal_i"].shape == given["valid_signal_o"].shape, "valid_signal_i / _o must have one length"
    kept = neighbor.__dict__.setdefault("_fgx_kernel_tables", [])
    tables = next((t for t in kept if _fits(t, given)), None)
    if tables is None:
        tables = SubMConv3dNeighborCache(neighbor_map=neighbor)
        kept.append(tables)
        del kept[:-4]
    for k, v in given.items():
        if getattr(tables, "_given_" + k, None) is None:
            tables["_given_" + k] = v
            tables[k] = v.contiguous()
    if "sorted_idx" in given and not hasattr(tables, "gray_code"):
        n, v = neighbor.shape
        gray = torch.empty((n,), dtype=torch.int32, device=neighbor.device)
        binary = torch.empty((n,), dtype=torch.int32, device=neighbor.device)
        with torch.cuda.device(neighbor.device):
            nat.check(nat.lib().fgx_mask_codes(nat.ptr(neighbor), nat.sz(n), C.c_int(v), nat.ptr(gray), nat.ptr(binary),
                                               nat.stream()))
        tables["gray_code"], tables["_binary_code"] = gray, binary
    return tables


def _check_fwd(input: torch.Tensor, weight: torch.Tensor, neighbor: torch.Tensor, transposed: bool = False) -> None:
    assert weight.ndim == 3 and weight.shape[1] == neighbor.shape[1], "weight must be [Co, V, Ci] with V = neighbor.shape[1]"
    assert input.shape[1] == (weight.shape[0] if transposed else weight.shape[2]), "Incompatible dimensions"
    assert input.is_contiguous(), "Matrix input must be contiguous"
    assert weight.is_contiguous(), "Matrix weight must be contiguous"
    assert neighbor.is_contiguous(), "Matrix neighbor must be contiguous"


# ---- submanifold convolution --------------------------------------------------------------------------------------

def _subm_fwd(input, weight, bias, neighbor, splitk: bool, sorted_idx=None) -> torch.Tensor:
    _check_fwd(input, weight, neighbor)
    assert input.shape[0] == neighbor.shape[0], "input and neighbor must have one row per voxel"
    tables = _tables_of(neighbor, sorted_idx=sorted_idx)
    return _gather_gemm(input, weight, bias, tables, 0, splitk, masked=sorted_idx is not None)


def _subm_bwd(grad_output, input, weight, bias, neighbor, splitk: bool, sorted_idx=None, pairs=(None, None, None)):
    assert grad_output.is_contiguous(), "Matrix grad_output must be contiguous"
    _check_fwd(input, weight, neighbor)
    assert input.shape[0] == neighbor.shape[0] and grad_output.shape[0] == neighbor.shape[0], \
        "input, grad_output and neighbor must have one row per voxel"
    tables = _tables_of(neighbor, sorted_idx=sorted_idx, valid_signal_i=pairs[0], valid_signal_o=pairs[1],
                        valid_signal_seg=pairs[2])
    v = weight.shape[1]
    grad_input = grad_weight = grad_bias = None
    if input.requires_grad:
        grad_input = _gather_gemm(grad_output, weight.detach(), None, tables, 1, splitk, masked=sorted_idx is not None)
    want_bias = bias is not None and bias.requires_grad
    if weight.requires_grad and want_bias:
        # an odd number of offsets has a centre that pairs every voxel with itself: the bias gradient rides along
        grad_weight, grad_bias = _wgrad(grad_output, input.detach(), tables, v, True, v // 2 if v % 2 else -1)
    elif weight.requires_grad:
        grad_weight = _wgrad(grad_output, input.detach(), tables, v)
    elif want_bias:
        grad_bias = _colsum(grad_output)
    return grad_input, grad_weight, grad_bias


def sparse_submanifold_conv_fwd_implicit_gemm(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                                              neighbor: torch.Tensor) -> torch.Tensor:
    """[N, Co] = convolution of input [N, Ci] over neighbor uint32 [N, V]; rows in natural order, every tile walks all V
    offsets (sparse_submanifold_conv_fwd_implicit_gemm.py:92-117)."""
    return _subm_fwd(input, weight, bias, neighbor, False)


def sparse_submanifold_conv_fwd_implicit_gemm_splitk(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                                                     neighbor: torch.Tensor, SPLITK: Optional[int] = None) -> torch.Tensor:
    """The same with the contraction split where the schedule table says so (..._fwd_implicit_gemm_splitk.py)."""
    return _subm_fwd(input, weight, bias, neighbor, True)


def sparse_submanifold_conv_fwd_masked_implicit_gemm(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                                                     neighbor: torch.Tensor, sorted_idx: torch.Tensor,
                                                     valid_kernel: Optional[Callable[[int], torch.Tensor]] = None,
                                                     valid_kernel_seg: Optional[Callable[[int], torch.Tensor]] = None) -> torch.Tensor:
    """Rows walked in the mask-sorted order `sorted_idx`, each tile skipping the offsets none of its rows has
    (..._fwd_masked_implicit_gemm.py:103-135)."""
    return _subm_fwd(input, weight, bias, neighbor, False, sorted_idx)


def sparse_submanifold_conv_fwd_masked_implicit_gemm_splitk(input: torch.Tensor, weight: torch.Tensor,
                                                            bias: Optional[torch.Tensor], neighbor: torch.Tensor,
                                                            sorted_idx: torch.Tensor,
                                                            valid_kernel: Optional[Callable[[int], torch.Tensor]] = None,
                                                            valid_kernel_seg: Optional[Callable[[int], torch.Tensor]] = None,
                                                            SPLITK: Optional[int] = None) -> torch.Tensor:
    """The default algorithm's forward kernel call (..._fwd_masked_implicit_gemm_splitk.py:139-184)."""
    return _subm_fwd(input, weight, bias, neighbor, True, sorted_idx)


def sparse_submanifold_conv_bwd_implicit_gemm(grad_output: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                                              bias: Optional[torch.Tensor], neighbor: torch.Tensor):
    """(grad_input, grad_weight, grad_bias) of the non-masked schedule (..._bwd_implicit_gemm.py:177-225)."""
    return _subm_bwd(grad_output, input, weight, bias, neighbor, False)


def sparse_submanifold_conv_bwd_implicit_gemm_splitk(grad_output: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                                                     bias: Optional[torch.Tensor], neighbor: torch.Tensor):
    return _subm_bwd(grad_output, input, weight, bias, neighbor, True)


def sparse_submanifold_conv_bwd_masked_implicit_gemm(grad_output: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                                                     bias: Optional[torch.Tensor], neighbor: torch.Tensor,
                                                     sorted_idx: torch.Tensor, valid_kernel=None, valid_kernel_seg=None,
                                                     valid_signal_i: Optional[torch.Tensor] = None,
                                                     valid_signal_o: Optional[torch.Tensor] = None,
                                                     valid_signal_seg: Optional[torch.Tensor] = None):
    """(grad_input, grad_weight, grad_bias); the weight gradient walks the caller's pair lists
    (..._bwd_masked_implicit_gemm.py:171-233).  Pair lists left out are derived from the map."""
    return _subm_bwd(grad_output, input, weight, bias, neighbor, False, sorted_idx,
                     (valid_signal_i, valid_signal_o, valid_signal_seg))


def sparse_submanifold_conv_bwd_masked_implicit_gemm_splitk(grad_output: torch.Tensor, input: torch.Tensor,
                                                            weight: torch.Tensor, bias: Optional[torch.Tensor],
                                                            neighbor: torch.Tensor, sorted_idx: torch.Tensor,
                                                            valid_kernel=None, valid_kernel_seg=None,
                                                            valid_signal_i: Optional[torch.Tensor] = None,
                                                            valid_signal_o: Optional[torch.Tensor] = None,
                                                            valid_signal_seg: Optional[torch.Tensor] = None):
    """The default algorithm's backward kernel call (..._bwd_masked_implicit_gemm_splitk.py:266-346)."""
    return _subm_bwd(grad_output, input, weight, bias, neighbor, True, sorted_idx,
                     (valid_signal_i, valid_signal_o, valid_signal_seg))


# ---- generic sparse convolution: neighbor [M, V] maps output rows to input rows ---------------------------------------

def _conv_fwd(input, weight, bias, neighbor, splitk: bool, sorted_idx=None, transposed: bool = False) -> torch.Tensor:
    _check_fwd(input, weight, neighbor, transposed)
    tables = _tables_of(neighbor, sorted_idx=sorted_idx)
    return _gather_gemm(input, weight, bias, tables, 2 if transposed else 0, splitk, masked=sorted_idx is not None)


def _conv_bwd(grad_output, input, weight, bias, neighbor, neighbor_bwd, splitk: bool, pairs=(None, None, None),
              sorted_idx_bwd=None):
    assert grad_output.is_contiguous(), "Matrix grad_output must be contiguous"
    _check_fwd(input, weight, neighbor)
    assert neighbor_bwd.is_contiguous(), "Matrix neighbor_bwd must be contiguous"
    assert input.shape[0] == neighbor_bwd.shape[0] and grad_output.shape[0] == neighbor.shape[0], \
        "input needs one row per row of neighbor_bwd, grad_output one per row of neighbor"
    grad_input = grad_weight = grad_bias = None
    if input.requires_grad:
        tables_bwd = _tables_of(neighbor_bwd, sorted_idx=sorted_idx_bwd)
        grad_input = _gather_gemm(grad_output, weight.detach(), None, tables_bwd, 2, splitk,
                                  masked=sorted_idx_bwd is not None)
    if weight.requires_grad:
        tables = _tables_of(neighbor, valid_signal_i=pairs[0], valid_signal_o=pairs[1], valid_signal_seg=pairs[2])
        grad_weight = _wgrad(grad_output, input.detach(), tables, weight.shape[1])
    if bias is not None and bias.requires_grad:
        grad_bias = _colsum(grad_output)
    return grad_input, grad_weight, grad_bias


def sparse_conv_fwd_implicit_gemm(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                                  neighbor: torch.Tensor) -> torch.Tensor:
    """[M, Co] from input [N, Ci] (sparse_conv_implicit_gemm.py:149-175)."""
    return _conv_fwd(input, weight, bias, neighbor, False)


def sparse_conv_fwd_implicit_gemm_splitk(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                                         neighbor: torch.Tensor, SPLITK: Optional[int] = None,
                                         TRANSPOSE_WEIGHT: bool = False) -> torch.Tensor:
    """TRANSPOSE_WEIGHT: contract over weight's first axis instead of its last, which is how the reference computes
    the input gradient through the backward map (sparse_conv_implicit_gemm_splitk.py:184-237)."""
    return _conv_fwd(input, weight, bias, neighbor, True, None, TRANSPOSE_WEIGHT)


def sparse_conv_fwd_masked_implicit_gemm(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                                         neighbor: torch.Tensor, sorted_idx: torch.Tensor, valid_kernel=None,
                                         valid_kernel_seg=None) -> torch.Tensor:
    return _conv_fwd(input, weight, bias, neighbor, False, sorted_idx)


def sparse_conv_fwd_masked_implicit_gemm_splitk(input: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor],
                                                neighbor: torch.Tensor, sorted_idx: torch.Tensor, valid_kernel=None,
                                                valid_kernel_seg=None, SPLITK: Optional[int] = None,
                                                TRANSPOSE_WEIGHT: bool = False) -> torch.Tensor:
    """sparse_conv_masked_implicit_gemm_splitk.py:226-273."""
    return _conv_fwd(input, weight, bias, neighbor, True, sorted_idx, TRANSPOSE_WEIGHT)


def sparse_conv_bwd_implicit_gemm(grad_output: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                                  bias: Optional[torch.Tensor], neighbor: torch.Tensor, neighbor_bwd: torch.Tensor):
    """sparse_conv_implicit_gemm.py:178-235."""
    return _conv_bwd(grad_output, input, weight, bias, neighbor, neighbor_bwd, False)


def sparse_conv_bwd_implicit_gemm_splitk(grad_output: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                                         bias: Optional[torch.Tensor], neighbor: torch.Tensor, neighbor_bwd: torch.Tensor):
    return _conv_bwd(grad_output, input, weight, bias, neighbor, neighbor_bwd, True)


def sparse_conv_bwd_masked_implicit_gemm(grad_output: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                                         bias: Optional[torch.Tensor], neighbor: torch.Tensor, neighbor_bwd: torch.Tensor,
                                         valid_signal_i: Optional[torch.Tensor] = None,
                                         valid_signal_o: Optional[torch.Tensor] = None,
                                         valid_signal_seg: Optional[torch.Tensor] = None,
                                         sorted_idx_bwd: Optional[torch.Tensor] = None, valid_kernel_bwd=None,
                                         valid_kernel_bwd_seg=None):
    """sorted_idx_bwd None: the input gradient walks the backward map in natural order, as in the reference
    (sparse_conv_masked_implicit_gemm.py:218-284)."""
    return _conv_bwd(grad_output, input, weight, bias, neighbor, neighbor_bwd, False,
                     (valid_signal_i, valid_signal_o, valid_signal_seg), sorted_idx_bwd)


def sparse_conv_bwd_masked_implicit_gemm_splitk(grad_output: torch.Tensor, input: torch.Tensor, weight: torch.Tensor,
                                                bias: Optional[torch.Tensor], neighbor: torch.Tensor,
                                                neighbor_bwd: torch.Tensor,
                                                valid_signal_i: Optional[torch.Tensor] = None,
                                                valid_signal_o: Optional[torch.Tensor] = None,
                                                valid_signal_seg: Optional[torch.Tensor] = None,
                                                sorted_idx_bwd: Optional[torch.Tensor] = None, valid_kernel_bwd=None,
                                                valid_kernel_bwd_seg=None):
    """sparse_conv_masked_implicit_gemm_splitk.py:342-416."""
    return _conv_bwd(grad_output, input, weight, bias, neighbor, neighbor_bwd, True,
                     (valid_signal_i, valid_signal_o, valid_signal_seg), sorted_idx_bwd)
