"""TEST INFRASTRUCTURE ONLY -- ctypes front-end of the C restatement in subm_ref.c.

Every function returns numpy arrays with the dtypes the reference's cache carries
(flex_gemm/ops/spconv/submanifold_conv3d.py:86-104): neighbor_map uint32 [N, V],
gray_code int32 [N], sorted_idx int64 [N], valid_signal_{i,o} uint32 [L],
valid_signal_seg uint32 [V+1], valid_kernel / valid_kernel_seg int32.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Dict, Optional, Sequence, Tuple

import numpy as np

from . import build as _build

EMPTY = np.uint32(0xFFFFFFFF)
_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        path = _build.build(force=False)
        _lib = C.CDLL(path)
        _lib.ref_fmix32.restype = C.c_uint32
        _lib.ref_fmix32.argtypes = [C.c_uint32]
        _lib.ref_fmix64.restype = C.c_uint64
        _lib.ref_fmix64.argtypes = [C.c_uint64]
        _lib.ref_tile_masks.restype = C.c_int64
    return _lib


def _p(a: Optional[np.ndarray]):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def fmix32(k: int) -> int:
    return int(lib().ref_fmix32(C.c_uint32(k & 0xFFFFFFFF)))


def fmix64(k: int) -> int:
    return int(lib().ref_fmix64(C.c_uint64(k & 0xFFFFFFFFFFFFFFFF)))


def key_bits_for(shape: Sequence[int]) -> int:
    """flex_gemm/ops/utils.py:9-12 -- uint32 keys iff B*W*H*D < 2^32."""
    b, _, w, h, d = shape
    vol = int(b) * int(w) * int(h) * int(d)
    if vol < 2 ** 32:
        return 32
    if vol < 2 ** 64:
        return 64
    raise ValueError("spatial size too large for a 64-bit key")


class HashTable:
    """Open-addressing table as the reference lays it out: keys[T] (all-ones = empty), vals[T] uint32."""

    def __init__(self, table_size: int, key_bits: int = 32):
        self.size = int(table_size)
        self.key_bits = key_bits
        self.keys = np.empty(self.size, dtype=np.uint32 if key_bits == 32 else np.uint64)
        self.vals = np.zeros(self.size, dtype=np.uint32)
        lib().ref_hash_init(_p(self.keys), C.c_int(key_bits), C.c_size_t(self.size))

    def insert_idx_as_val(self, coords: np.ndarray, W: int, H: int, D: int) -> None:
        coords = np.ascontiguousarray(coords, dtype=np.int32)
        lib().ref_hash_insert_idx_as_val(_p(self.keys), C.c_int(self.key_bits), _p(self.vals), C.c_size_t(self.size),
                                         _p(coords), C.c_size_t(coords.shape[0]), C.c_int(W), C.c_int(H), C.c_int(D))

    def insert_3d(self, coords: np.ndarray, values: np.ndarray, W: int, H: int, D: int) -> None:
        coords = np.ascontiguousarray(coords, dtype=np.int32)
        values = np.ascontiguousarray(values, dtype=np.uint32)
        lib().ref_hash_insert_3d(_p(self.keys), C.c_int(self.key_bits), _p(self.vals), C.c_size_t(self.size),
                                 _p(coords), _p(values), C.c_size_t(coords.shape[0]),
                                 C.c_int(W), C.c_int(H), C.c_int(D))

    def lookup_3d(self, coords: np.ndarray, W: int, H: int, D: int) -> np.ndarray:
        coords = np.ascontiguousarray(coords, dtype=np.int32)
        out = np.empty(coords.shape[0], dtype=np.uint32)
        lib().ref_hash_lookup_3d(_p(self.keys), C.c_int(self.key_bits), _p(self.vals), C.c_size_t(self.size),
                                 _p(coords), C.c_size_t(coords.shape[0]), C.c_int(W), C.c_int(H), C.c_int(D), _p(out))
        return out


def neighbor_map(coords: np.ndarray, shape: Sequence[int], kernel_size=(3, 3, 3), dilation=(1, 1, 1),
                 hashmap_ratio: float = 2.0) -> np.ndarray:
    """Hash build + 14-probe/mirror lookup exactly as the reference sequences them
    (submanifold_conv3d.py:57-67 -> subm_neighbor_map.cu:104-162)."""
    coords = np.ascontiguousarray(coords, dtype=np.int32)
    n = coords.shape[0]
    _, _, W, H, D = [int(s) for s in shape]
    kb = key_bits_for(shape)
    table = HashTable(int(hashmap_ratio * n), kb)
    table.insert_idx_as_val(coords, W, H, D)
    V = kernel_size[0] * kernel_size[1] * kernel_size[2]
    out = np.empty((n, V), dtype=np.uint32)
    lib().ref_subm_neighbor_map(_p(table.keys), C.c_int(kb), _p(table.vals), C.c_size_t(table.size),
                                _p(coords), C.c_size_t(n), C.c_int(W), C.c_int(H), C.c_int(D),
                                C.c_int(kernel_size[0]), C.c_int(kernel_size[1]), C.c_int(kernel_size[2]),
                                C.c_int(dilation[0]), C.c_int(dilation[1]), C.c_int(dilation[2]), _p(out))
    return out


def gray_binary(nmap: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    nmap = np.ascontiguousarray(nmap, dtype=np.uint32)
    n, V = nmap.shape
    gray = np.empty(n, dtype=np.int32)
    binary = np.empty(n, dtype=np.int32)
    lib().ref_gray_binary(_p(nmap), C.c_size_t(n), C.c_int(V), _p(gray), _p(binary))
    return gray, binary


def sorted_idx_canonical(binary: np.ndarray) -> np.ndarray:
    """The reference sorts with an unstable argsort (migemm_neighmap_pp.cu:79,221), so ties are
    unspecified there; the canonical representative used for comparisons is the stable order."""
    return np.argsort(binary.astype(np.int32), kind="stable").astype(np.int64)


def pair_lists(nmap: np.ndarray) -> Tuple[np.ndarray, np.ndarray, np.ndarray]:
    """(valid_signal_i, valid_signal_o, valid_signal_seg)."""
    nmap = np.ascontiguousarray(nmap, dtype=np.uint32)
    n, V = nmap.shape
    seg = np.empty(V + 1, dtype=np.uint32)
    lib().ref_pair_lists(_p(nmap), C.c_size_t(n), C.c_int(V), None, None, _p(seg))
    L = int(seg[V])
    sig_i = np.empty(L, dtype=np.uint32)
    sig_o = np.empty(L, dtype=np.uint32)
    lib().ref_pair_lists(_p(nmap), C.c_size_t(n), C.c_int(V), _p(sig_i), _p(sig_o), _p(seg))
    return sig_i, sig_o, seg


def tile_masks(gray: np.ndarray, sorted_idx: np.ndarray, block: int) -> Tuple[np.ndarray, np.ndarray]:
    """(valid_kernel, valid_kernel_seg) for row-tile size `block`."""
    gray = np.ascontiguousarray(gray, dtype=np.int32)
    sorted_idx = np.ascontiguousarray(sorted_idx, dtype=np.int64)
    n = gray.shape[0]
    nb = (n + block - 1) // block
    seg = np.empty(nb + 1, dtype=np.int32)
    total = lib().ref_tile_masks(_p(gray), _p(sorted_idx), C.c_size_t(n), C.c_int(block), None, _p(seg))
    vk = np.empty(int(total), dtype=np.int32)
    lib().ref_tile_masks(_p(gray), _p(sorted_idx), C.c_size_t(n), C.c_int(block), _p(vk), _p(seg))
    return vk, seg


def neighbor_cache(coords: np.ndarray, shape: Sequence[int], kernel_size=(3, 3, 3), dilation=(1, 1, 1),
                   needs_grad: bool = True, blocks: Sequence[int] = ()) -> Dict[str, np.ndarray]:
    """All tables of the masked-implicit-GEMM cache (submanifold_conv3d.py:73-104)."""
    nmap = neighbor_map(coords, shape, kernel_size, dilation)
    gray, binary = gray_binary(nmap)
    out = {"neighbor_map": nmap, "gray_code": gray, "binary_code": binary,
           "sorted_idx": sorted_idx_canonical(binary)}
    if needs_grad:
        out["valid_signal_i"], out["valid_signal_o"], out["valid_signal_seg"] = pair_lists(nmap)
    for b in blocks:
        out[f"valid_kernel_{b}"], out[f"valid_kernel_seg_{b}"] = tile_masks(gray, out["sorted_idx"], b)
    return out
