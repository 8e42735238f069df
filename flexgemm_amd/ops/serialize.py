"""Space-filling-curve codes of voxel coordinates: the MI355X stand-in for `flex_gemm.ops.serialize`
(reference: flex_gemm/ops/serialize.py:7-72).  Same names, arguments, code dtype rule and errors; the work runs in
flexgemm_amd/csrc/serialize.hip.  Tensors must live on the GPU: there is no host implementation."""
import ctypes as C
from typing import Literal

import torch

from .. import _native as nat

_MODE_CODE = {"z_order": 1, "hilbert": 2}


def _bit_length(shape) -> int:
    _, _, a, b, c = [int(s) for s in shape]
    return (max(a, b, c) - 1).bit_length()


def _mode_code(mode: str, verb: str) -> int:
    if mode not in _MODE_CODE:
        raise ValueError(f"Unknown {verb} mode: {mode}")
    return _MODE_CODE[mode]


@torch.no_grad()
def encode_seq(coords: torch.Tensor, shape: torch.Size, mode: Literal["z_order", "hilbert"] = "z_order") -> torch.Tensor:
    """Codes of [N, 4] int32 (b, x, y, z) coordinates along the chosen curve.

    Args:
        coords: [N, 4] coordinates.
        shape (torch.Size): shape of the sparse tensor in NCWHD order; the largest spatial extent fixes the bits per axis.
        mode: 'z_order' or 'hilbert'.
    Returns int32 codes when batch bits + 3 * bits per axis <= 32, int64 codes up to 64 bits, ValueError beyond
    (reference: serialize.py:21-33)."""
    assert coords.shape[-1] == 4 and coords.ndim == 2, "Input coordinates must be of shape [N, 4]"
    code = _mode_code(mode, "encoding")
    bit_length = _bit_length(shape)
    total_bit_length = (int(shape[0]) - 1).bit_length() + 3 * bit_length
    if total_bit_length <= 32:
        dtype, code_bits = torch.int32, 32
    elif total_bit_length <= 64:
        dtype, code_bits = torch.int64, 64
    else:
        raise ValueError(f"Spatial dimensions are too large: {shape}")
    if not coords.is_cuda:
        raise NotImplementedError("encode_seq runs on the GPU only: move coords to the device")
    assert coords.dtype == torch.int32, "Unsupported coords dtype. Expect int32"
    coords = coords.contiguous()
    codes = torch.empty(coords.shape[0], dtype=dtype, device=coords.device)
    with torch.cuda.device(coords.device):
        nat.check(nat.lib().fgx_serialize_encode(C.c_int(code), nat.ptr(coords), nat.sz(coords.shape[0]), C.c_int(bit_length),
                                                 C.c_int(code_bits), nat.ptr(codes), nat.stream()))
    return codes


def decode_seq(code: torch.Tensor, shape: torch.Size, mode: Literal["z_order", "hilbert"] = "z_order") -> torch.Tensor:
    """[N, 4] int32 (b, x, y, z) coordinates of int32 / int64 codes (reference: serialize.py:46-72)."""
    assert code.ndim == 1, "Input code must be of shape [N]"
    mode_code = _mode_code(mode, "decoding")
    bit_length = _bit_length(shape)
    if code.dtype == torch.int32:
        code_bits = 32
    elif code.dtype == torch.int64:
        code_bits = 64
    else:
        raise RuntimeError("Unsupported input type")
    if not code.is_cuda:
        raise NotImplementedError("decode_seq runs on the GPU only: move the codes to the device")
    code = code.contiguous()
    coords = torch.empty((code.shape[0], 4), dtype=torch.int32, device=code.device)
    with torch.cuda.device(code.device):
        nat.check(nat.lib().fgx_serialize_decode(C.c_int(mode_code), nat.ptr(code), nat.sz(code.shape[0]), C.c_int(bit_length),
                                                 C.c_int(code_bits), nat.ptr(coords), nat.stream()))
    return coords


def reorder_coords(coords: torch.Tensor, bit_length: int, batch_bits: int, mode_code: int) -> torch.Tensor:
    """coords sorted along the curve (1 = z-order, 2 = Hilbert): one encode, one radix sort, one decode on the device."""
    n = coords.shape[0]
    code_bits = 32 if batch_bits + 3 * bit_length <= 32 else 64
    if batch_bits + 3 * bit_length > 64:
        raise ValueError("The spatial size is too large. Require total bit length < 64.")
    out = torch.empty_like(coords)
    if n == 0:
        return out
    L = nat.lib()
    with torch.cuda.device(coords.device):
        ws = nat.workspace(L.fgx_serialize_reorder_workspace_bytes(nat.sz(n), C.c_int(code_bits)), coords.device)
        nat.check(L.fgx_serialize_reorder_coords(C.c_int(mode_code), nat.ptr(coords), nat.sz(n), C.c_int(bit_length),
                                                 C.c_int(batch_bits), C.c_int(code_bits), nat.ptr(ws), nat.sz(ws.numel()),
                                                 nat.ptr(out), nat.stream()))
    return out
