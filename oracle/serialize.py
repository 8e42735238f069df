"""CPU restatement of the reference's voxel serialisation (space-filling-curve codes).  TEST INFRASTRUCTURE ONLY:
nothing shipped may import this module.

What is restated
  * z-order (Morton) codes: flex_gemm/kernels/cuda/serialize/z_order.h:22-40 -- bit i of x, y, z lands on code bit
    3i+2, 3i+1, 3i; the batch index sits above the 3*bit_length spatial bits.
  * Hilbert codes: flex_gemm/kernels/cuda/serialize/hilbert.h:22-118 -- J. Skilling, "Programming the Hilbert curve",
    AIP Conf. Proc. 707 (2004): axes -> "transpose" form (undo excess work, Gray encode), whose bits are then
    interleaved exactly like a Morton code with axis 0 (x) as the most significant of each triple.
  * code width and bit_length: flex_gemm/ops/serialize.py:21-31 (int32 when batch bits + 3*bit_length <= 32,
    else int64; bit_length = (max extent - 1).bit_length()).

Here bits are interleaved one at a time in a loop, not with the reference's magic-mask shuffles, so that the two
formulations check each other through the HIP kernels.

Pinning (tests/test_oracle_serialize.py): hand-derived first-order Hilbert octant order; for orders 1..4 the codes of
the full cube are a bijection onto 0..8^k-1, consecutive codes are face-adjacent cells, code 0 is the origin and the
last code is (2^k-1, 0, 0); Morton codes against per-bit Python-integer brute force and hand values; decode inverts
encode.  One divergence from the reference is deliberate: for 64-bit z-order codes the reference shifts the 32-bit
batch index without widening it (z_order.h:29), which drops the batch for bit_length >= 11; here the batch is kept
(the behaviour hilbert.h:73 has and the round trip of tests/serialize.py needs).
"""
import numpy as np

MODES = ("z_order", "hilbert")


def bit_lengths(shape):
    """(spatial bit_length, total bits) of a [N, C, W, H, D] shape -- flex_gemm/ops/serialize.py:21-26."""
    n, _, w, h, d = [int(s) for s in shape]
    bl = (max(w, h, d) - 1).bit_length()
    return bl, (n - 1).bit_length() + 3 * bl


def code_dtype(shape):
    _, total = bit_lengths(shape)
    if total <= 32:
        return np.int32
    if total <= 64:
        return np.int64
    raise ValueError(f"Spatial dimensions are too large: {tuple(shape)}")


def _interleave(p0, p1, p2, bit_length):
    code = np.zeros(p0.shape, dtype=np.uint64)
    for i in range(bit_length):
        code |= ((p0 >> np.uint64(i)) & np.uint64(1)) << np.uint64(3 * i + 2)
        code |= ((p1 >> np.uint64(i)) & np.uint64(1)) << np.uint64(3 * i + 1)
        code |= ((p2 >> np.uint64(i)) & np.uint64(1)) << np.uint64(3 * i)
    return code


def _deinterleave(code, bit_length):
    p = [np.zeros(code.shape, dtype=np.uint64) for _ in range(3)]
    for i in range(bit_length):
        p[0] |= ((code >> np.uint64(3 * i + 2)) & np.uint64(1)) << np.uint64(i)
        p[1] |= ((code >> np.uint64(3 * i + 1)) & np.uint64(1)) << np.uint64(i)
        p[2] |= ((code >> np.uint64(3 * i)) & np.uint64(1)) << np.uint64(i)
    return p


def _axes_to_transpose(x, y, z, bit_length):
    """Skilling's AxestoTranspose on three uint64 arrays (hilbert.h:23-56)."""
    p = [x.copy(), y.copy(), z.copy()]
    if bit_length == 0:
        return p
    top = 1 << (bit_length - 1)
    q = top
    while q > 1:
        low = np.uint64(q - 1)
        for i in range(3):
            hit = (p[i] & np.uint64(q)) != 0
            swap = np.where(hit, np.uint64(0), (p[0] ^ p[i]) & low)
            p[0] = np.where(hit, p[0] ^ low, p[0] ^ swap)
            # for i == 0 the swap term is zero, so the second update is the identity, as in the scalar form
            p[i] = np.where(hit, p[i], p[i] ^ swap) if i else p[0]
        q >>= 1
    p[1] ^= p[0]
    p[2] ^= p[1]
    t = np.zeros_like(p[0])
    q = top
    while q > 1:
        t ^= np.where((p[2] & np.uint64(q)) != 0, np.uint64(q - 1), np.uint64(0))
        q >>= 1
    return [c ^ t for c in p]


def _transpose_to_axes(p, bit_length):
    """Skilling's TransposetoAxes (hilbert.h:79-113)."""
    p = [c.copy() for c in p]
    if bit_length == 0:
        return p
    t = p[2] >> np.uint64(1)
    p[2] ^= p[1]
    p[1] ^= p[0]
    p[0] ^= t
    q = 2
    while q != (1 << bit_length):
        low = np.uint64(q - 1)
        for i in (2, 1, 0):
            hit = (p[i] & np.uint64(q)) != 0
            swap = np.where(hit, np.uint64(0), (p[0] ^ p[i]) & low)
            p[0] = np.where(hit, p[0] ^ low, p[0] ^ swap)
            p[i] = np.where(hit, p[i], p[i] ^ swap) if i else p[0]
        q <<= 1
    return p


def encode(coords, bit_length, mode="z_order", dtype=np.int64):
    """codes[n] of coords int[n, 4] = (b, x, y, z); `dtype` int32 or int64 as code_dtype() chose."""
    if mode not in MODES:
        raise ValueError(f"Unknown encoding mode: {mode}")
    c = np.asarray(coords).astype(np.int64).astype(np.uint64).reshape(-1, 4)
    x, y, z = c[:, 1], c[:, 2], c[:, 3]
    if mode == "hilbert":
        x, y, z = _axes_to_transpose(x, y, z, bit_length)
    code = _interleave(x, y, z, bit_length) | (c[:, 0] << np.uint64(3 * bit_length))
    if np.dtype(dtype) == np.int32:
        return (code & np.uint64(0xFFFFFFFF)).astype(np.uint32).view(np.int32)
    return code.view(np.int64)


def decode(codes, bit_length, mode="z_order"):
    """coords int32[n, 4] of codes int32/int64[n]."""
    if mode not in MODES:
        raise ValueError(f"Unknown decoding mode: {mode}")
    codes = np.asarray(codes)
    if codes.dtype == np.int32:
        u = codes.view(np.uint32).astype(np.uint64)
    else:
        u = codes.astype(np.int64).view(np.uint64)
    spatial = u & np.uint64((1 << (3 * bit_length)) - 1)
    p = _deinterleave(spatial, bit_length)
    if mode == "hilbert":
        p = _transpose_to_axes(p, bit_length)
    b = u >> np.uint64(3 * bit_length)
    return np.stack([b, p[0], p[1], p[2]], axis=1).astype(np.int64).astype(np.int32)


def encode_seq(coords, shape, mode="z_order"):
    """flex_gemm/ops/serialize.py:7-43."""
    bl, _ = bit_lengths(shape)
    return encode(coords, bl, mode, code_dtype(shape))


def decode_seq(codes, shape, mode="z_order"):
    """flex_gemm/ops/serialize.py:46-72."""
    bl, _ = bit_lengths(shape)
    return decode(codes, bl, mode)


def reorder_coords(coords, bit_length, mode):
    """coords sorted by their (unsigned) code: the order the reference leaves output coordinates in under
    SerializationMode.Z_ORDER / HILBERT (sparse_neighbor_map.cu:156-187 with utils.h:47-107)."""
    code = encode(coords, bit_length, mode, np.int64).view(np.uint64)
    return np.asarray(coords)[np.argsort(code, kind="stable")]
