"""The reference's native module `flex_gemm.kernels.cuda` (pybind11, flex_gemm/kernels/cuda/ext.cpp:10-36) under its own
function names and argument orders, for code and tests that call it directly (tests/hashmap.py:38,56,
ops/serialize.py:35-70, ops/spconv/*.py).  Every function is a thin host wrapper over the C ABI of
include/flexgemm_hip.h: tensors must live on the GPU, outputs are allocated here as torch tensors, work is enqueued on
torch's current stream.  The two grid-sample builders are another operator and raise NotImplementedError.
"""
from __future__ import annotations

import ctypes as C
from typing import Tuple

import torch

from .. import _native as nat

_BITS = {torch.uint32: 32, torch.uint64: 64, torch.int32: 32, torch.int64: 64}


def _bits(t: torch.Tensor, what: str) -> int:
    if t.dtype not in _BITS:
        raise RuntimeError(f"Unsupported {what} dtype {t.dtype}")
    return _BITS[t.dtype]


def _on_gpu(*tensors: torch.Tensor) -> torch.device:
    dev = tensors[0].device
    for t in tensors:
        if not t.is_cuda:
            raise NotImplementedError("flex_gemm.kernels.cuda runs on the GPU only: move the tensors to the device")
        if t.device != dev:
            raise RuntimeError("all tensors must live on one device")
    return dev


# ---- hash table (flex_gemm/kernels/cuda/hash/api.h:30-113) ---------------------------------------------------------

def hashmap_insert(hashmap_keys: torch.Tensor, hashmap_values: torch.Tensor, keys: torch.Tensor, values: torch.Tensor) -> None:
    dev = _on_gpu(hashmap_keys, hashmap_values, keys, values)
    assert keys.dtype == hashmap_keys.dtype and values.dtype == hashmap_values.dtype, "key / value dtypes must match the table's"
    keys, values = keys.contiguous(), values.contiguous()
    with torch.cuda.device(dev):
        nat.check(nat.lib().fgx_hash_insert(nat.ptr(hashmap_keys), C.c_int(_bits(hashmap_keys, "key")), nat.ptr(hashmap_values),
                                            C.c_int(_bits(hashmap_values, "value")), nat.sz(hashmap_keys.shape[0]), nat.ptr(keys),
                                            nat.ptr(values), nat.sz(keys.shape[0]), nat.stream()))


def hashmap_lookup(hashmap_keys: torch.Tensor, hashmap_values: torch.Tensor, keys: torch.Tensor) -> torch.Tensor:
    dev = _on_gpu(hashmap_keys, hashmap_values, keys)
    assert keys.dtype == hashmap_keys.dtype, "key dtype must match the table's"
    keys = keys.contiguous()
    out = torch.empty((keys.shape[0],), dtype=hashmap_values.dtype, device=dev)
    with torch.cuda.device(dev):
        nat.check(nat.lib().fgx_hash_lookup(nat.ptr(hashmap_keys), C.c_int(_bits(hashmap_keys, "key")), nat.ptr(hashmap_values),
                                            C.c_int(_bits(hashmap_values, "value")), nat.sz(hashmap_keys.shape[0]), nat.ptr(keys),
                                            nat.ptr(out), nat.sz(keys.shape[0]), nat.stream()))
    return out


def hashmap_insert_3d(hashmap_keys: torch.Tensor, hashmap_values: torch.Tensor, coords: torch.Tensor, values: torch.Tensor,
                      W: int, H: int, D: int) -> None:
    dev = _on_gpu(hashmap_keys, hashmap_values, coords, values)
    assert coords.dtype == torch.int32 and coords.ndim == 2 and coords.shape[1] == 4, "coords must be int32 [N, 4]"
    assert values.dtype == hashmap_values.dtype, "value dtype must match the table's"
    coords, values = coords.contiguous(), values.contiguous()
    with torch.cuda.device(dev):
        nat.check(nat.lib().fgx_hash_insert_3d(nat.ptr(hashmap_keys), C.c_int(_bits(hashmap_keys, "key")), nat.ptr(hashmap_values),
                                               C.c_int(_bits(hashmap_values, "value")), nat.sz(hashmap_keys.shape[0]),
                                               nat.ptr(coords), nat.ptr(values), nat.sz(coords.shape[0]), C.c_int(W), C.c_int(H),
                                               C.c_int(D), nat.stream()))


def hashmap_lookup_3d(hashmap_keys: torch.Tensor, hashmap_values: torch.Tensor, coords: torch.Tensor, W: int, H: int,
                      D: int) -> torch.Tensor:
    dev = _on_gpu(hashmap_keys, hashmap_values, coords)
    assert coords.dtype == torch.int32 and coords.ndim == 2 and coords.shape[1] == 4, "coords must be int32 [N, 4]"
    coords = coords.contiguous()
    out = torch.empty((coords.shape[0],), dtype=hashmap_values.dtype, device=dev)
    with torch.cuda.device(dev):
        nat.check(nat.lib().fgx_hash_lookup_3d(nat.ptr(hashmap_keys), C.c_int(_bits(hashmap_keys, "key")), nat.ptr(hashmap_values),
                                               C.c_int(_bits(hashmap_values, "value")), nat.sz(hashmap_keys.shape[0]),
                                               nat.ptr(coords), nat.ptr(out), nat.sz(coords.shape[0]), C.c_int(W), C.c_int(H),
                                               C.c_int(D), nat.stream()))
    return out


def hashmap_insert_3d_idx_as_val(hashmap_keys: torch.Tensor, hashmap_values: torch.Tensor, coords: torch.Tensor, W: int, H: int,
                                 D: int) -> None:
    dev = _on_gpu(hashmap_keys, hashmap_values, coords)
    assert coords.dtype == torch.int32 and coords.ndim == 2 and coords.shape[1] == 4, "coords must be int32 [N, 4]"
    coords = coords.contiguous()
    with torch.cuda.device(dev):
        nat.check(nat.lib().fgx_hash_insert_3d_idx_as_val(
            nat.ptr(hashmap_keys), C.c_int(_bits(hashmap_keys, "key")), nat.ptr(hashmap_values),
            C.c_int(_bits(hashmap_values, "value")), nat.sz(hashmap_keys.shape[0]), nat.ptr(coords), nat.sz(coords.shape[0]),
            C.c_int(W), C.c_int(H), C.c_int(D), nat.stream()))


# ---- serialisation (flex_gemm/kernels/cuda/serialize/api.h:22-76) --------------------------------------------------

def _encode(mode: int, coords: torch.Tensor, bit_length: int, codes: torch.Tensor) -> None:
    dev = _on_gpu(coords, codes)
    assert coords.dtype == torch.int32 and coords.ndim == 2 and coords.shape[1] == 4, "coords must be int32 [N, 4]"
    if codes.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("Unsupported output type")
    coords = coords.contiguous()
    with torch.cuda.device(dev):
        nat.check(nat.lib().fgx_serialize_encode(C.c_int(mode), nat.ptr(coords), nat.sz(coords.shape[0]), C.c_int(int(bit_length)),
                                                 C.c_int(_bits(codes, "code")), nat.ptr(codes), nat.stream()))


def _decode(mode: int, codes: torch.Tensor, bit_length: int) -> torch.Tensor:
    dev = _on_gpu(codes)
    if codes.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("Unsupported input type")
    codes = codes.contiguous()
    coords = torch.empty((codes.shape[0], 4), dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        nat.check(nat.lib().fgx_serialize_decode(C.c_int(mode), nat.ptr(codes), nat.sz(codes.shape[0]), C.c_int(int(bit_length)),
                                                 C.c_int(_bits(codes, "code")), nat.ptr(coords), nat.stream()))
    return coords


def z_order_encode(coords: torch.Tensor, bit_length: int, codes: torch.Tensor) -> None:
    _encode(1, coords, bit_length, codes)


def z_order_decode(codes: torch.Tensor, bit_length: int) -> torch.Tensor:
    return _decode(1, codes, bit_length)


def hilbert_encode(coords: torch.Tensor, bit_length: int, codes: torch.Tensor) -> None:
    _encode(2, coords, bit_length, codes)


def hilbert_decode(codes: torch.Tensor, bit_length: int) -> torch.Tensor:
    return _decode(2, codes, bit_length)


# ---- grid sample: another operator ----------------------------------------------------------------------------------

def hashmap_build_grid_sample_3d_nearest_neighbor_map(*args, **kwargs):
    raise NotImplementedError("grid sample is not part of this build (sparse convolution path only)")


def hashmap_build_grid_sample_3d_trilinear_neighbor_map_weight(*args, **kwargs):
    raise NotImplementedError("grid sample is not part of this build (sparse convolution path only)")


# ---- convolution tables (flex_gemm/kernels/cuda/spconv/*.h) ---------------------------------------------------------

def _check_map(neighbor_map: torch.Tensor) -> None:
    assert neighbor_map.dtype == torch.uint32 and neighbor_map.ndim == 2, "neighbor_map must be uint32 [N, V]"
    assert neighbor_map.shape[1] <= 32, "Currently, the max kernel volume is 32 because kernel mask is encoded as uint32"


def hashmap_build_submanifold_conv_neighbour_map(hashmap_keys: torch.Tensor, hashmap_vals: torch.Tensor, coords: torch.Tensor,
                                                 W: int, H: int, D: int, Kw: int, Kh: int, Kd: int, Dw: int, Dh: int,
                                                 Dd: int) -> torch.Tensor:
    """uint32 [N, Kw*Kh*Kd] neighbor map; fills the caller's (initialised) table with the voxels on the way
    (subm_neighbor_map.h:40-47, .cu:104-162)."""
    dev = _on_gpu(hashmap_keys, hashmap_vals, coords)
    assert hashmap_vals.dtype == torch.uint32, "the neighbor-map builder keeps row numbers: hashmap values must be uint32"
    assert hashmap_keys.shape[0] == hashmap_vals.shape[0], "key and value tables must have one length"
    hashmap_insert_3d_idx_as_val(hashmap_keys, hashmap_vals, coords, W, H, D)
    coords = coords.contiguous()
    n = coords.shape[0]
    out = torch.empty((n, Kw * Kh * Kd), dtype=torch.uint32, device=dev)
    with torch.cuda.device(dev):
        nat.check(nat.lib().fgx_subm_neighbor_map(
            nat.ptr(hashmap_keys), C.c_int(_bits(hashmap_keys, "key")), nat.ptr(hashmap_vals), nat.sz(hashmap_keys.shape[0]),
            nat.ptr(coords), nat.sz(n), C.c_int(W), C.c_int(H), C.c_int(D), C.c_int(Kw), C.c_int(Kh), C.c_int(Kd),
            C.c_int(Dw), C.c_int(Dh), C.c_int(Dd), nat.ptr(out), None, None, nat.stream()))
    return out


def neighbor_map_post_process_for_masked_implicit_gemm_1_no_bwd(neighbor_map: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """(gray_code int32 [N], sorted_idx int64 [N])   (migemm_neighmap_pp.h:33-44)."""
    from ..ops.spconv.submanifold_conv3d import _codes_and_order
    _on_gpu(neighbor_map)
    _check_map(neighbor_map)
    gray, _, order = _codes_and_order(neighbor_map.contiguous(), None, None)
    return gray, order


def neighbor_map_post_process_for_masked_implicit_gemm_1(neighbor_map: torch.Tensor):
    """(gray_code, sorted_idx, valid_signal_i, valid_signal_o, valid_signal_seg)   (migemm_neighmap_pp.h:46-58)."""
    from ..ops.spconv.submanifold_conv3d import _codes_and_order, _pair_lists
    _on_gpu(neighbor_map)
    _check_map(neighbor_map)
    nmap = neighbor_map.contiguous()
    gray, _, order = _codes_and_order(nmap, None, None)
    pairs = _pair_lists(nmap, gray, exact=True)
    return gray, order, pairs["sig_i"], pairs["sig_o"], pairs["seg"]


def neighbor_map_post_process_for_masked_implicit_gemm_2(gray_code: torch.Tensor, sorted_idx: torch.Tensor,
                                                         block_size: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """(valid_kernel int32 [sum], valid_kernel_seg int32 [ceil(N / block_size) + 1])   (migemm_neighmap_pp.h:60-70)."""
    dev = _on_gpu(gray_code, sorted_idx)
    assert gray_code.dtype == torch.int32 and gray_code.ndim == 1, "gray_code must be int32 [N]"
    assert sorted_idx.dtype == torch.int64 and sorted_idx.shape == gray_code.shape, "sorted_idx must be int64 [N]"
    if int(block_size) < 1:
        raise ValueError(f"block_size must be positive, got {block_size}")
    n = gray_code.shape[0]
    block_size = int(block_size)
    nb = (n + block_size - 1) // block_size
    code = torch.empty((nb,), dtype=torch.int32, device=dev)
    seg = torch.empty((nb + 1,), dtype=torch.int32, device=dev)
    L = nat.lib()
    with torch.cuda.device(dev):
        ws = nat.workspace(L.fgx_tile_workspace_bytes(nat.sz(n), C.c_int(block_size)), dev)
        nat.check(L.fgx_tile_codes(nat.ptr(gray_code.contiguous()), nat.ptr(sorted_idx.contiguous()), nat.sz(n), C.c_int(block_size),
                                   nat.ptr(code), nat.ptr(seg), nat.ptr(ws), nat.sz(ws.numel()), nat.stream()))
        total = int(seg[-1].item())
        vk = torch.empty((total,), dtype=torch.int32, device=dev)
        if total:
            nat.check(L.fgx_tile_fill(nat.ptr(code), nat.ptr(seg), nat.sz(nb), nat.ptr(vk), nat.stream()))
    return vk, seg


def _out_coords(in_coords: torch.Tensor, serialize_mode: int, B, W, H, D, Kw, Kh, Kd, Sw, Sh, Sd, Pw, Ph, Pd, Dw, Dh, Dd):
    from ..ops.spconv.sparse_conv3d import SparseConv3dFunction
    _on_gpu(in_coords)
    if serialize_mode not in (0, 1, 2):
        raise RuntimeError("Unsupported serialize mode.")
    return SparseConv3dFunction._get_output_coords(in_coords.contiguous(), torch.Size([B, 0, W, H, D]), (Kw, Kh, Kd),
                                                   (Sw, Sh, Sd), (Pw, Ph, Pd), (Dw, Dh, Dd), serialization_mode=serialize_mode)


def hashmap_build_sparse_conv_out_coords(in_coords: torch.Tensor, hashmap_ratio: float, serialize_mode: int, B: int, W: int,
                                         H: int, D: int, Kw: int, Kh: int, Kd: int, Sw: int, Sh: int, Sd: int, Pw: int,
                                         Ph: int, Pd: int, Dw: int, Dh: int, Dd: int) -> torch.Tensor:
    """int32 [L, 4] output coordinates in the order of `serialize_mode` (sparse_neighbor_map.h:42-56).  One streaming
    pass (candidate keys, sort, unique) serves this and the expand-unique entry; hashmap_ratio has nothing to size."""
    del hashmap_ratio
    return _out_coords(in_coords, serialize_mode, B, W, H, D, Kw, Kh, Kd, Sw, Sh, Sd, Pw, Ph, Pd, Dw, Dh, Dd)


def expand_unique_build_sparse_conv_out_coords(in_coords: torch.Tensor, serialize_mode: int, B: int, W: int, H: int, D: int,
                                               Kw: int, Kh: int, Kd: int, Sw: int, Sh: int, Sd: int, Pw: int, Ph: int,
                                               Pd: int, Dw: int, Dh: int, Dd: int) -> torch.Tensor:
    """The same list by the reference's other algorithm name (sparse_neighbor_map.h:78-91)."""
    return _out_coords(in_coords, serialize_mode, B, W, H, D, Kw, Kh, Kd, Sw, Sh, Sd, Pw, Ph, Pd, Dw, Dh, Dd)


def hashmap_build_sparse_conv_neighbour_map(in_coords: torch.Tensor, out_coords: torch.Tensor, hashmap_ratio: float,
                                            include_bwd: bool, B: int, W: int, H: int, D: int, Kw: int, Kh: int, Kd: int,
                                            Sw: int, Sh: int, Sd: int, Pw: int, Ph: int, Pd: int, Dw: int, Dh: int,
                                            Dd: int):
    """(neighbor_map uint32 [L, V], neighbor_map_bwd uint32 [M, V] -- an empty tensor when include_bwd is false)
    (sparse_neighbor_map.h:88-131)."""
    from ..ops.spconv.sparse_conv3d import _build_maps
    dev = _on_gpu(in_coords, out_coords)
    fwd, bwd, _, _ = _build_maps(in_coords.contiguous(), out_coords.contiguous(), torch.Size([B, 0, W, H, D]), (Kw, Kh, Kd),
                                 (Sw, Sh, Sd), (Pw, Ph, Pd), (Dw, Dh, Dd), bool(include_bwd), False,
                                 hashmap_ratio=hashmap_ratio)
    if bwd is None:
        bwd = torch.empty((0,), dtype=torch.uint32, device=dev)
    return fwd, bwd
