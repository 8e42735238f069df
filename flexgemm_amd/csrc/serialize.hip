// Space-filling-curve codes of voxel coordinates for gfx950: z-order (Morton) and Hilbert, encode / decode, and the
// "sort coordinates along the curve" pass the generic sparse convolution uses for its output coordinates.
//
// Semantics follow flex_gemm/kernels/cuda/serialize/z_order.h:22-40 and hilbert.h:22-118: x, y, z contribute bit i to
// code bits 3i+2, 3i+1, 3i; the batch index sits above the 3*bit_length spatial bits; the Hilbert code is the Morton
// code of Skilling's "transpose" of the point (J. Skilling, Programming the Hilbert curve, 2004).  The batch index is
// widened before it is shifted for both curves (the reference's z-order path shifts it as a 32-bit value, which loses
// it for 64-bit codes with bit_length >= 11).
//
// All three passes are streaming: 16 bytes of coordinates and 4 or 8 bytes of code per voxel, one thread per voxel,
// 16-byte vector accesses on the coordinate side.  The bit shuffles are a few dozen integer operations per voxel and
// hide behind the memory traffic.
#include <cstring>
#include <string.h>

#include <rocprim/rocprim.hpp>

#include "fgx_common.h"

namespace fgx {
namespace {

constexpr int kBlock = 256;
constexpr int kZOrder = 1, kHilbert = 2;      // SerializationMode values of flex_gemm/ops/spconv/__init__.py:20-24

// Bits i with (i / run) % 3 == 0: runs of `run` ones, two runs of zeros between them.
template <typename T>
constexpr T run_mask(int run) {
    T m = 0;
    for (int i = 0; i < (int)(8 * sizeof(T)); ++i)
        if ((i / run) % 3 == 0) m |= (T)1 << i;
    return m;
}

// Moves bit i of v to bit 3i by doubling: each step pushes the upper half of every run two run-lengths up.
template <typename T, int RUN>
__host__ __device__ __forceinline__ T spread_step(T v) {
    constexpr T m = run_mask<T>(RUN);
    v = (v | (v << (2 * RUN))) & m;
    if constexpr (RUN > 1) v = spread_step<T, RUN / 2>(v);
    return v;
}

template <typename T>
__host__ __device__ __forceinline__ T spread3(T v) {
    return spread_step<T, (int)(2 * sizeof(T))>(v);      // first run length: 8 for 32-bit codes, 16 for 64-bit ones
}

// Inverse: collects bits 0, 3, 6, ... of v into the low bits.
template <typename T, int RUN>
__host__ __device__ __forceinline__ T gather_step(T v) {
    constexpr T m = run_mask<T>(2 * RUN > (int)(8 * sizeof(T)) ? (int)(8 * sizeof(T)) : 2 * RUN);
    v = (v | (v >> (2 * RUN))) & m;
    if constexpr (4 * RUN <= (int)(4 * sizeof(T))) v = gather_step<T, 2 * RUN>(v);
    return v;
}

template <typename T>
__host__ __device__ __forceinline__ T gather3(T v) {
    return gather_step<T, 1>(v & run_mask<T>(1));
}

// One level of Skilling's exchange/invert for axis value a against axis 0 (p0): if the level bit of a is set, the low
// bits of p0 are inverted, otherwise the low bits in which p0 and a differ are exchanged.
__host__ __device__ __forceinline__ void fold_axis(uint32_t& p0, uint32_t& a, uint32_t q, uint32_t low) {
    const bool set = (a & q) != 0;
    const uint32_t t = set ? 0u : ((p0 ^ a) & low);
    p0 ^= set ? low : t;
    a ^= t;
}

__host__ __device__ __forceinline__ void fold_axis0(uint32_t& p0, uint32_t q, uint32_t low) {
    if (p0 & q) p0 ^= low;
}

__host__ __device__ __forceinline__ void axes_to_transpose(uint32_t& x, uint32_t& y, uint32_t& z, int bits) {
    if (bits <= 0) return;
    const uint32_t top = 1u << (bits - 1);
    for (uint32_t q = top; q > 1; q >>= 1) {
        const uint32_t low = q - 1;
        fold_axis0(x, q, low);
        fold_axis(x, y, q, low);
        fold_axis(x, z, q, low);
    }
    y ^= x;
    z ^= y;
    uint32_t t = 0;
    for (uint32_t q = top; q > 1; q >>= 1)
        if (z & q) t ^= q - 1;
    x ^= t;
    y ^= t;
    z ^= t;
}

__host__ __device__ __forceinline__ void transpose_to_axes(uint32_t& x, uint32_t& y, uint32_t& z, int bits) {
    if (bits <= 0) return;
    const uint32_t t = z >> 1;
    z ^= y;
    y ^= x;
    x ^= t;
    const uint32_t end = 1u << bits;       // bits <= 21
    for (uint32_t q = 2; q != end; q <<= 1) {
        const uint32_t low = q - 1;
        fold_axis(x, z, q, low);
        fold_axis(x, y, q, low);
        fold_axis0(x, q, low);
    }
}

template <typename T>
__host__ __device__ __forceinline__ T spatial_mask(int bits) {
    return bits == 0 ? (T)0 : (T)(~(T)0) >> (8 * sizeof(T) - 3 * bits);
}

template <typename T, int MODE>
__host__ __device__ __forceinline__ T encode_one(int4 c, int bits) {
    const uint32_t keep = bits >= 32 ? 0xFFFFFFFFu : ((1u << bits) - 1u);
    uint32_t x = (uint32_t)c.y & keep, y = (uint32_t)c.z & keep, z = (uint32_t)c.w & keep;
    if (MODE == kHilbert) axes_to_transpose(x, y, z, bits);
    const T spatial = (spread3<T>((T)x) << 2) | (spread3<T>((T)y) << 1) | spread3<T>((T)z);
    const int shift = 3 * bits;
    const T batch = shift >= (int)(8 * sizeof(T)) ? (T)0 : (T)(uint32_t)c.x << shift;
    return (spatial & spatial_mask<T>(bits)) | batch;
}

template <typename T, int MODE>
__host__ __device__ __forceinline__ int4 decode_one(T code, int bits) {
    const T spatial = code & spatial_mask<T>(bits);
    uint32_t x = (uint32_t)gather3<T>(spatial >> 2), y = (uint32_t)gather3<T>(spatial >> 1), z = (uint32_t)gather3<T>(spatial);
    if (MODE == kHilbert) transpose_to_axes(x, y, z, bits);
    const int shift = 3 * bits;
    const uint32_t b = shift >= (int)(8 * sizeof(T)) ? 0u : (uint32_t)(code >> shift);
    return make_int4((int)b, (int)x, (int)y, (int)z);
}

template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock) encode_kernel(const int32_t* __restrict__ coords, size_t n, int bits,
                                                        T* __restrict__ codes) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    codes[i] = encode_one<T, MODE>(reinterpret_cast<const int4*>(coords)[i], bits);
}

template <typename T, int MODE>
__global__ void __launch_bounds__(kBlock) decode_kernel(const T* __restrict__ codes, size_t n, int bits,
                                                        int32_t* __restrict__ coords) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    reinterpret_cast<int4*>(coords)[i] = decode_one<T, MODE>(codes[i], bits);
}

template <typename T>
int launch_encode(int mode, const int32_t* coords, size_t n, int bits, T* codes, hipStream_t s) {
    if (mode == kZOrder)
        encode_kernel<T, kZOrder><<<cdiv(n, kBlock), kBlock, 0, s>>>(coords, n, bits, codes);
    else
        encode_kernel<T, kHilbert><<<cdiv(n, kBlock), kBlock, 0, s>>>(coords, n, bits, codes);
    FGX_CHECK_LAUNCH("fgx_serialize_encode");
    return FGX_OK;
}

template <typename T>
int launch_decode(int mode, const T* codes, size_t n, int bits, int32_t* coords, hipStream_t s) {
    if (mode == kZOrder)
        decode_kernel<T, kZOrder><<<cdiv(n, kBlock), kBlock, 0, s>>>(codes, n, bits, coords);
    else
        decode_kernel<T, kHilbert><<<cdiv(n, kBlock), kBlock, 0, s>>>(codes, n, bits, coords);
    FGX_CHECK_LAUNCH("fgx_serialize_decode");
    return FGX_OK;
}

int check_mode_bits(const char* who, int mode, int bit_length, int code_bits) {
    FGX_CHECK_ARG(mode == kZOrder || mode == kHilbert, "%s: mode must be 1 (z-order) or 2 (Hilbert), got %d", who, mode);
    FGX_CHECK_ARG(code_bits == 32 || code_bits == 64, "%s: code_bits must be 32 or 64, got %d", who, code_bits);
    FGX_CHECK_ARG(bit_length >= 0 && 3 * bit_length <= code_bits, "%s: bit_length %d does not fit %d-bit codes", who, bit_length,
                  code_bits);
    return FGX_OK;
}

struct ReorderLayout {
    size_t codes_a, codes_b, temp, temp_bytes, total;
};

template <typename T>
size_t sort_temp_bytes(size_t n) {
    size_t bytes = 0;
    (void)rocprim::radix_sort_keys(nullptr, bytes, (const T*)nullptr, (T*)nullptr, n ? n : 1, 0u, (unsigned)(8 * sizeof(T)),
                                   (hipStream_t)0);
    return bytes;
}

ReorderLayout reorder_layout(size_t n, int code_bits) {
    ReorderLayout L{};
    const size_t es = code_bits / 8, m = n ? n : 1;
    size_t off = 0;
    L.codes_a = off;
    off = align_up(off + m * es, 256);
    L.codes_b = off;
    off = align_up(off + m * es, 256);
    L.temp = off;
    L.temp_bytes = code_bits == 32 ? sort_temp_bytes<uint32_t>(n) : sort_temp_bytes<uint64_t>(n);
    L.total = off + align_up(L.temp_bytes, 256);
    return L;
}

template <typename T>
int reorder_impl(int mode, const int32_t* coords, size_t n, int bits, unsigned used_bits, char* ws, const ReorderLayout& L,
                 int32_t* out_coords, hipStream_t s) {
    T* a = (T*)(ws + L.codes_a);
    T* b = (T*)(ws + L.codes_b);
    int rc = launch_encode<T>(mode, coords, n, bits, a, s);
    if (rc != FGX_OK) return rc;
    size_t temp_bytes = L.temp_bytes;
    FGX_CHECK_HIP(rocprim::radix_sort_keys(ws + L.temp, temp_bytes, (const T*)a, b, n, 0u, used_bits, s));
    return launch_decode<T>(mode, b, n, bits, out_coords, s);
}

}  // namespace
}  // namespace fgx

using namespace fgx;

extern "C" {

int fgx_serialize_encode(int mode, const int32_t* coords, size_t n, int bit_length, int code_bits, void* codes,
                         fgx_stream_t stream) {
    int rc = check_mode_bits("fgx_serialize_encode", mode, bit_length, code_bits);
    if (rc != FGX_OK) return rc;
    if (n == 0) return FGX_OK;
    FGX_CHECK_ARG(coords && codes, "fgx_serialize_encode: null buffer");
    FGX_CHECK_ARG(((uintptr_t)coords & 15) == 0, "fgx_serialize_encode: coords must be 16-byte aligned");
    FGX_CHECK_ARG(((uintptr_t)codes & (code_bits / 8 - 1)) == 0, "fgx_serialize_encode: codes are misaligned");
    hipStream_t s = (hipStream_t)stream;
    return code_bits == 32 ? launch_encode<uint32_t>(mode, coords, n, bit_length, (uint32_t*)codes, s)
                           : launch_encode<uint64_t>(mode, coords, n, bit_length, (uint64_t*)codes, s);
}

int fgx_serialize_decode(int mode, const void* codes, size_t n, int bit_length, int code_bits, int32_t* coords,
                         fgx_stream_t stream) {
    int rc = check_mode_bits("fgx_serialize_decode", mode, bit_length, code_bits);
    if (rc != FGX_OK) return rc;
    if (n == 0) return FGX_OK;
    FGX_CHECK_ARG(coords && codes, "fgx_serialize_decode: null buffer");
    FGX_CHECK_ARG(((uintptr_t)coords & 15) == 0, "fgx_serialize_decode: coords must be 16-byte aligned");
    FGX_CHECK_ARG(((uintptr_t)codes & (code_bits / 8 - 1)) == 0, "fgx_serialize_decode: codes are misaligned");
    hipStream_t s = (hipStream_t)stream;
    return code_bits == 32 ? launch_decode<uint32_t>(mode, (const uint32_t*)codes, n, bit_length, coords, s)
                           : launch_decode<uint64_t>(mode, (const uint64_t*)codes, n, bit_length, coords, s);
}

size_t fgx_serialize_reorder_workspace_bytes(size_t n, int code_bits) {
    if (code_bits != 32 && code_bits != 64) return 0;
    return reorder_layout(n, code_bits).total;
}

int fgx_serialize_reorder_coords(int mode, const int32_t* coords, size_t n, int bit_length, int batch_bits, int code_bits,
                                 void* workspace, size_t workspace_bytes, int32_t* out_coords, fgx_stream_t stream) {
    int rc = check_mode_bits("fgx_serialize_reorder_coords", mode, bit_length, code_bits);
    if (rc != FGX_OK) return rc;
    FGX_CHECK_ARG(batch_bits >= 0 && batch_bits + 3 * bit_length <= code_bits,
                  "fgx_serialize_reorder_coords: %d batch bits + 3 * %d do not fit %d-bit codes", batch_bits, bit_length, code_bits);
    if (n == 0) return FGX_OK;
    FGX_CHECK_ARG(coords && out_coords && workspace, "fgx_serialize_reorder_coords: null buffer");
    FGX_CHECK_ARG(coords != out_coords, "fgx_serialize_reorder_coords: in-place reordering is not supported");
    FGX_CHECK_ARG((((uintptr_t)coords | (uintptr_t)out_coords) & 15) == 0,
                  "fgx_serialize_reorder_coords: coordinate buffers must be 16-byte aligned");
    FGX_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fgx_serialize_reorder_coords: workspace must be 256-byte aligned");
    const ReorderLayout L = reorder_layout(n, code_bits);
    FGX_CHECK_ARG(workspace_bytes >= L.total, "fgx_serialize_reorder_coords: workspace of %zu bytes, need %zu", workspace_bytes,
                  L.total);
    unsigned used = (unsigned)(batch_bits + 3 * bit_length);
    if (used == 0) used = 1;
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)workspace;
    return code_bits == 32 ? reorder_impl<uint32_t>(mode, coords, n, bit_length, used, ws, L, out_coords, s)
                           : reorder_impl<uint64_t>(mode, coords, n, bit_length, used, ws, L, out_coords, s);
}

}  // extern "C"
