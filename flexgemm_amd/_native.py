"""ctypes binding of libflexgemm_hip.so (the C ABI declared in include/flexgemm_hip.h).

The library is mandatory: nothing in this package falls back to another implementation when
it is missing.  Device pointers, sizes and the current HIP stream are taken from torch tensors;
torch itself is only the allocator and the stream owner.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

import torch

# (FGX_LIB_PATH: another build of the same library, e.g. one compiled with different kernel parameters)
_LIB_PATH = os.environ.get("FGX_LIB_PATH") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "_lib", "libflexgemm_hip.so")
_lib: Optional[C.CDLL] = None

FGX_F16, FGX_BF16, FGX_F32 = 0, 1, 2
DTYPE_CODE = {torch.float16: FGX_F16, torch.bfloat16: FGX_BF16, torch.float32: FGX_F32}
ACT_NONE, ACT_RELU = 0, 1          # FGX_ACT_* of the public header
PASS_FWD, PASS_DGRAD, PASS_WGRAD = 0, 1, 2

# every symbol the header declares; the CPU-side test checks that the library exports each of them
EXPORTS = [
    "fgx_abi_version", "fgx_last_error", "fgx_set_phase_hook",
    "fgx_hash_init", "fgx_hash_insert_3d_idx_as_val", "fgx_hash_insert", "fgx_hash_lookup",
    "fgx_hash_insert_3d", "fgx_hash_lookup_3d",
    "fgx_subm_neighbor_map", "fgx_subm_neighbor_map_sorted_workspace_bytes", "fgx_subm_neighbor_map_sorted", "fgx_coords_key_order", "fgx_mask_codes",
    "fgx_sort_workspace_bytes", "fgx_sort_by_code", "fgx_locality_workspace_bytes", "fgx_locality_order", "fgx_locality_order_grid",
    "fgx_pair_workspace_bytes", "fgx_pair_count", "fgx_pair_fill", "fgx_subm_cache_workspace_bytes", "fgx_subm_cache_build",
    "fgx_tile_workspace_bytes", "fgx_tile_codes", "fgx_tile_fill",
    "fgx_table_lookup", "fgx_weight_panel_bytes", "fgx_pack_weight",
    "fgx_conv_scratch_bytes", "fgx_conv_gather_gemm", "fgx_conv_gather_gemm_act", "fgx_conv_gather_gemm_act_mask",
    "fgx_relu_mask_apply", "fgx_conv_gather_gemm_stream_act_mask",
    "fgx_gather_plan_count", "fgx_gather_plan_fill", "fgx_conv_gather_gemm_stream", "fgx_conv_gather_gemm_stream_act",
    "fgx_conv_gather_gemm_stream_groups", "fgx_gather_item_order_workspace_bytes", "fgx_gather_item_order",
    "fgx_wgrad_scratch_bytes", "fgx_wgrad_block_bounds_count", "fgx_wgrad_block_bounds", "fgx_conv_wgrad",
    "fgx_wgrad_item_lists_count", "fgx_wgrad_item_lists", "fgx_conv_wgrad_lists",
    "fgx_zorder_rows", "fgx_narrow_plan_bytes", "fgx_narrow_plan", "fgx_conv_narrow_gemm", "fgx_narrow_wgrad_scratch_bytes", "fgx_conv_narrow_wgrad",
    "fgx_wgrad_sweep_plan_bytes", "fgx_wgrad_sweep_plan", "fgx_wgrad_sweep_scratch_bytes", "fgx_conv_wgrad_sweep",
    "fgx_wgrad_sweep_giveup_words", "fgx_wgrad_sweep_reduce",
    "fgx_colsum_scratch_bytes", "fgx_colsum", "fgx_colsum_static_prepare", "fgx_colsum_static_max_cols", "fgx_colsum_static",
    "fgx_spconv_out_dims", "fgx_spconv_out_coords_workspace_bytes", "fgx_spconv_out_coords_keys",
    "fgx_spconv_out_coords_decode", "fgx_spconv_neighbor_map",
    "fgx_spconv_neighbor_map_sorted_workspace_bytes", "fgx_spconv_neighbor_map_sorted",
    "fgx_serialize_encode", "fgx_serialize_decode", "fgx_serialize_reorder_workspace_bytes",
    "fgx_serialize_reorder_coords",
]


# Optional profiling hook: callable(name, phase) with phase "start"/"stop", invoked on the launching thread right
# before / after the named native call is enqueued (bench.py records HIP events on the current stream from it).
EVENT_HOOK = None


def mark(name: str, phase: str) -> None:
    if EVENT_HOOK is not None:
        EVENT_HOOK(name, phase)


PHASE_HOOK_T = C.CFUNCTYPE(None, C.c_char_p, C.c_void_p)
_phase_hook_ref = None      # keeps the ctypes trampoline alive while the library holds its address


def set_phase_hook(fn) -> None:
    """fn(phase_name: str, stream: int) is called by the library's multi-kernel calls right before each of their phases
    is enqueued ("" after the last one); None switches it off (fgx_set_phase_hook)."""
    global _phase_hook_ref
    if fn is None:
        lib().fgx_set_phase_hook(PHASE_HOOK_T(0))
        _phase_hook_ref = None
        return
    cb = PHASE_HOOK_T(lambda name, stream: fn(name.decode() if name else "", stream))
    lib().fgx_set_phase_hook(cb)
    _phase_hook_ref = cb


class Schedule(C.Structure):
    _fields_ = [("tile_rows", C.c_int), ("tile_cols", C.c_int), ("slab_bytes", C.c_int), ("splitk", C.c_int),
                ("block_rows", C.c_int), ("stream", C.c_int)]


class NativeError(RuntimeError):
    pass


def lib_path() -> str:
    return _LIB_PATH


def lib() -> C.CDLL:
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise NativeError(
                f"{_LIB_PATH} is missing: build it with `python -m flexgemm_amd.build` "
                "(hipcc --offload-arch=gfx950).  There is no fallback implementation.")
        L = C.CDLL(_LIB_PATH)
        L.fgx_last_error.restype = C.c_char_p
        for name in ("fgx_sort_workspace_bytes", "fgx_locality_workspace_bytes", "fgx_pair_workspace_bytes", "fgx_tile_workspace_bytes",
                     "fgx_weight_panel_bytes", "fgx_conv_scratch_bytes", "fgx_wgrad_scratch_bytes",
                     "fgx_colsum_scratch_bytes", "fgx_spconv_out_coords_workspace_bytes",
                     "fgx_subm_neighbor_map_sorted_workspace_bytes", "fgx_wgrad_block_bounds_count", "fgx_wgrad_item_lists_count", "fgx_narrow_plan_bytes", "fgx_narrow_wgrad_scratch_bytes",
                     "fgx_spconv_neighbor_map_sorted_workspace_bytes", "fgx_serialize_reorder_workspace_bytes",
                     "fgx_gather_item_order_workspace_bytes", "fgx_subm_cache_workspace_bytes", "fgx_wgrad_sweep_plan_bytes", "fgx_wgrad_sweep_scratch_bytes", "fgx_wgrad_sweep_giveup_words"):
            getattr(L, name).restype = C.c_size_t
        _lib = L
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        msg = lib().fgx_last_error().decode("utf-8", "replace")
        if rc == -1:
            raise ValueError(msg)
        if rc == -3:
            raise NotImplementedError(msg)
        raise NativeError(msg)


def ptr(t: Optional[torch.Tensor]) -> C.c_void_p:
    """Device address of a tensor for the C entry points, which take plain pointers and assume dense rows."""
    if t is None:
        return C.c_void_p(0)
    if not t.is_contiguous():
        raise ValueError(f"a strided view (shape {tuple(t.shape)}, strides {t.stride()}) was about to be passed as a plain pointer")
    return C.c_void_p(t.data_ptr())


def stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def sz(x: int) -> C.c_size_t:
    return C.c_size_t(int(x))


def workspace(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


_schedules: dict = {}        # (pass, dtype, n, ci, co, v) -> bytes of the library's answer (a pure function of the key)


def table_lookup(pass_kind: int, dtype: torch.dtype, n: int, ci: int, co: int, v: int) -> Schedule:
    """The library's schedule for a pass and shape.  Answers are remembered per key (the hot path asks on every call);
    every caller gets a Schedule of its own, so changing its fields changes nothing for the next one."""
    key = (pass_kind, dtype, int(n), int(ci), int(co), int(v))
    raw = _schedules.get(key)
    if raw is None:
        s = Schedule()
        check(lib().fgx_table_lookup(C.c_int(pass_kind), C.c_int(DTYPE_CODE[dtype]), sz(n), C.c_int(ci), C.c_int(co),
                                     C.c_int(v), C.byref(s)))
        if len(_schedules) > 4096:
            _schedules.clear()
        raw = _schedules[key] = bytes(s)
    return Schedule.from_buffer_copy(raw)
