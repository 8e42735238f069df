// Output coordinates and neighbor maps of the generic sparse convolution (stride / padding / dilation) for gfx950.
//
// Output coordinates.  The reference inserts every (input voxel, kernel position) candidate into a hash set, compacts
// the table and sorts the survivors (flex_gemm/kernels/cuda/spconv/sparse_neighbor_map.cu:19-131), or expands, and
// calls a library unique (:197-345).  Both leave the coordinates sorted by their flattened key.  Here the pass is
// pure streaming work: one coalesced write of all candidate keys (an unreachable candidate becomes the key one past
// the grid, so it sorts last), one radix sort over just the bits a key can have, one unique.  No atomics, no table.
//
// Neighbor maps.  One half-wave (32 lanes) owns one output voxel, lane v probes kernel position v in the hash table
// of the input voxels, the 4*V-byte row goes out as one coalesced store, and the backward map -- which input row
// feeds which output row at position v -- is scattered from the same lane (the reference does both from one thread
// per (voxel, position), sparse_neighbor_map.cu:431-467).
#include <cstring>
#include <string.h>

#include <rocprim/rocprim.hpp>

#include "fgx_common.h"
#include "hash_device.h"

namespace fgx {
namespace {

constexpr int kBlock = 256;

struct ConvGeom {
    int W, H, D;        // input grid
    int Wo, Ho, Do;     // output grid
    int Kw, Kh, Kd, V;
    int Sw, Sh, Sd;
    int Pw, Ph, Pd;
    int Dw, Dh, Dd;
};

int out_extent(int n, int k, int s, int p, int d) {
    const long long num = (long long)n + 2ll * p - (long long)d * (k - 1) - 1;
    // floor division, as Python's // in the reference's size formula
    const long long q = num >= 0 ? num / s : -((-num + s - 1) / s);
    return (int)(q + 1);
}

// floor(a / s) and "s divides a" for s > 0 and any a
__device__ __forceinline__ bool exact_div(int a, int s, int& q) {
    q = a / s;
    int r = a - q * s;
    return r == 0;      // C division truncates, but a zero remainder means the same under either convention
}

// key of candidate (voxel i, kernel position v): the flattened output coordinate, or `vol` (one past the largest key)
template <typename K>
__global__ void __launch_bounds__(kBlock) expand_keys_kernel(const int32_t* __restrict__ coords, size_t n, ConvGeom g,
                                                             K vol, K* __restrict__ keys) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= n * (size_t)g.V) return;
    const size_t i = t / g.V;
    const int v = (int)(t % g.V);
    const int4 c = reinterpret_cast<const int4*>(coords)[i];
    const int kx = v / (g.Kh * g.Kd), ky = v / g.Kd % g.Kh, kz = v % g.Kd;
    int ox, oy, oz;
    bool ok = exact_div(c.y + g.Pw - kx * g.Dw, g.Sw, ox);
    ok &= exact_div(c.z + g.Ph - ky * g.Dh, g.Sh, oy);
    ok &= exact_div(c.w + g.Pd - kz * g.Dd, g.Sd, oz);
    ok = ok && ox >= 0 && ox < g.Wo && oy >= 0 && oy < g.Ho && oz >= 0 && oz < g.Do;
    keys[t] = ok ? (K)flat_key(c.x, ox, oy, oz, g.Wo, g.Ho, g.Do) : vol;
}

// drops the "unreachable" key, which sorts last when present
template <typename K>
__global__ void trim_count_kernel(const K* __restrict__ unique_keys, K vol, uint64_t* __restrict__ count) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        uint64_t c = *count;
        if (c > 0 && unique_keys[c - 1] == vol) *count = c - 1;
    }
}

template <typename K>
__global__ void __launch_bounds__(kBlock) decode_keys_kernel(const K* __restrict__ keys, size_t count, int Wo, int Ho,
                                                             int Do, int32_t* __restrict__ out_coords) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= count) return;
    uint64_t k = (uint64_t)keys[t];
    int4 c;
    c.w = (int)(k % (uint64_t)Do);
    k /= (uint64_t)Do;
    c.z = (int)(k % (uint64_t)Ho);
    k /= (uint64_t)Ho;
    c.y = (int)(k % (uint64_t)Wo);
    c.x = (int)(k / (uint64_t)Wo);
    reinterpret_cast<int4*>(out_coords)[t] = c;
}

__global__ void __launch_bounds__(kBlock) fill_u32_kernel(uint32_t* p, size_t count, uint32_t value) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (; i < count; i += stride) p[i] = value;
}

__device__ __forceinline__ uint32_t gray_decode(uint32_t g) {
    g ^= g >> 16;
    g ^= g >> 8;
    g ^= g >> 4;
    g ^= g >> 2;
    g ^= g >> 1;
    return g;
}

// Half-wave per output voxel, V <= 32.
template <typename K>
__global__ void __launch_bounds__(kBlock) spconv_map_halfwave_kernel(
    const K* __restrict__ keys, const uint32_t* __restrict__ vals, size_t table, const int32_t* __restrict__ out_coords,
    size_t n_out, ConvGeom g, uint32_t* __restrict__ map_fwd, uint32_t* __restrict__ map_bwd, int32_t* __restrict__ gray,
    int32_t* __restrict__ binary) {
    const size_t o = ((size_t)blockIdx.x * kBlock + threadIdx.x) >> 5;
    const int v = threadIdx.x & 31;
    const bool active = o < n_out && v < g.V;
    uint32_t value = FGX_EMPTY32;
    if (active) {
        const int4 c = reinterpret_cast<const int4*>(out_coords)[o];
        const int x = c.y * g.Sw - g.Pw + v / (g.Kh * g.Kd) * g.Dw;
        const int y = c.z * g.Sh - g.Ph + v / g.Kd % g.Kh * g.Dh;
        const int z = c.w * g.Sd - g.Pd + v % g.Kd * g.Dd;
        if (x >= 0 && x < g.W && y >= 0 && y < g.H && z >= 0 && z < g.D)
            value = probe_lookup(keys, vals, (K)flat_key(c.x, x, y, z, g.W, g.H, g.D), table);
        map_fwd[o * (size_t)g.V + v] = value;
        if (map_bwd != nullptr && value != FGX_EMPTY32) map_bwd[(size_t)value * g.V + v] = (uint32_t)o;
    }
    if (gray != nullptr) {
        const unsigned long long found = __ballot(active && value != FGX_EMPTY32);
        const uint32_t m = (uint32_t)(found >> (threadIdx.x & 32));
        if (v == 0 && o < n_out) {
            gray[o] = (int32_t)m;
            binary[o] = (int32_t)gray_decode(m);
        }
    }
}

// Any V: one thread per (output voxel, kernel position).
template <typename K>
__global__ void __launch_bounds__(kBlock) spconv_map_flat_kernel(
    const K* __restrict__ keys, const uint32_t* __restrict__ vals, size_t table, const int32_t* __restrict__ out_coords,
    size_t n_out, ConvGeom g, uint32_t* __restrict__ map_fwd, uint32_t* __restrict__ map_bwd) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= n_out * (size_t)g.V) return;
    const size_t o = t / g.V;
    const int v = (int)(t % g.V);
    const int4 c = reinterpret_cast<const int4*>(out_coords)[o];
    const int x = c.y * g.Sw - g.Pw + v / (g.Kh * g.Kd) * g.Dw;
    const int y = c.z * g.Sh - g.Ph + v / g.Kd % g.Kh * g.Dh;
    const int z = c.w * g.Sd - g.Pd + v % g.Kd * g.Dd;
    uint32_t value = FGX_EMPTY32;
    if (x >= 0 && x < g.W && y >= 0 && y < g.H && z >= 0 && z < g.D)
        value = probe_lookup(keys, vals, (K)flat_key(c.x, x, y, z, g.W, g.H, g.D), table);
    map_fwd[t] = value;
    if (map_bwd != nullptr && value != FGX_EMPTY32) map_bwd[(size_t)value * g.V + v] = (uint32_t)o;
}

struct CoordsLayout {
    size_t keys_a, keys_b, temp, temp_bytes, total;
};

template <typename K>
size_t coords_temp_bytes(size_t m) {
    size_t sort_bytes = 0, uniq_bytes = 0;
    (void)rocprim::radix_sort_keys(nullptr, sort_bytes, (const K*)nullptr, (K*)nullptr, m ? m : 1, 0u, (unsigned)(8 * sizeof(K)),
                                   (hipStream_t)0);
    (void)rocprim::unique(nullptr, uniq_bytes, (const K*)nullptr, (K*)nullptr, (uint64_t*)nullptr, m ? m : 1,
                          rocprim::equal_to<K>(), (hipStream_t)0);
    return sort_bytes > uniq_bytes ? sort_bytes : uniq_bytes;
}

CoordsLayout coords_layout(size_t n_in, int V, int key_bits) {
    CoordsLayout L{};
    const size_t m = n_in * (size_t)V, es = key_bits / 8;
    size_t off = 0;
    L.keys_a = off;
    off = align_up(off + (m ? m : 1) * es, 256);
    L.keys_b = off;
    off = align_up(off + (m ? m : 1) * es, 256);
    L.temp = off;
    L.temp_bytes = key_bits == 32 ? coords_temp_bytes<uint32_t>(m) : coords_temp_bytes<uint64_t>(m);
    L.total = off + align_up(L.temp_bytes, 256);
    return L;
}

int check_geom(const char* who, int W, int H, int D, int Kw, int Kh, int Kd, int Sw, int Sh, int Sd, int Pw, int Ph, int Pd,
               int Dw, int Dh, int Dd, ConvGeom* g) {
    FGX_CHECK_ARG(W > 0 && H > 0 && D > 0, "%s: grid extents must be positive", who);
    FGX_CHECK_ARG(Kw > 0 && Kh > 0 && Kd > 0, "%s: kernel sizes must be positive, got (%d,%d,%d)", who, Kw, Kh, Kd);
    FGX_CHECK_ARG(Sw > 0 && Sh > 0 && Sd > 0, "%s: strides must be positive, got (%d,%d,%d)", who, Sw, Sh, Sd);
    FGX_CHECK_ARG(Dw > 0 && Dh > 0 && Dd > 0, "%s: dilations must be positive, got (%d,%d,%d)", who, Dw, Dh, Dd);
    FGX_CHECK_ARG(Pw >= 0 && Ph >= 0 && Pd >= 0, "%s: paddings must not be negative, got (%d,%d,%d)", who, Pw, Ph, Pd);
    const long long V = (long long)Kw * Kh * Kd;
    FGX_CHECK_ARG(V <= 1 << 20, "%s: kernel volume too large", who);
    *g = ConvGeom{W, H, D, out_extent(W, Kw, Sw, Pw, Dw), out_extent(H, Kh, Sh, Ph, Dh), out_extent(D, Kd, Sd, Pd, Dd),
                  Kw, Kh, Kd, (int)V, Sw, Sh, Sd, Pw, Ph, Pd, Dw, Dh, Dd};
    return FGX_OK;
}

unsigned bit_length(uint64_t x) {
    unsigned b = 0;
    while (x) {
        ++b;
        x >>= 1;
    }
    return b;
}

template <typename K>
int out_coords_keys_impl(const int32_t* coords, size_t n_in, const ConvGeom& g, uint64_t vol, char* ws, const CoordsLayout& L,
                         uint64_t* count, hipStream_t s) {
    K* keys_a = (K*)(ws + L.keys_a);
    K* keys_b = (K*)(ws + L.keys_b);
    const size_t m = n_in * (size_t)g.V;
    expand_keys_kernel<K><<<cdiv(m, kBlock), kBlock, 0, s>>>(coords, n_in, g, (K)vol, keys_a);
    FGX_CHECK_LAUNCH("fgx_spconv_out_coords_keys(expand)");
    size_t temp_bytes = L.temp_bytes;
    unsigned end_bit = bit_length(vol);          // keys are <= vol
    if (end_bit == 0) end_bit = 1;
    FGX_CHECK_HIP(rocprim::radix_sort_keys(ws + L.temp, temp_bytes, (const K*)keys_a, keys_b, m, 0u, end_bit, s));
    temp_bytes = L.temp_bytes;
    FGX_CHECK_HIP(rocprim::unique(ws + L.temp, temp_bytes, (const K*)keys_b, keys_a, count, m, rocprim::equal_to<K>(), s));
    trim_count_kernel<K><<<1, 64, 0, s>>>(keys_a, (K)vol, count);
    FGX_CHECK_LAUNCH("fgx_spconv_out_coords_keys(trim)");
    return FGX_OK;
}

}  // namespace
}  // namespace fgx

using namespace fgx;

extern "C" {

int fgx_spconv_out_dims(int W, int H, int D, int Kw, int Kh, int Kd, int Sw, int Sh, int Sd, int Pw, int Ph, int Pd, int Dw,
                        int Dh, int Dd, int* Wo, int* Ho, int* Do) {
    ConvGeom g;
    int rc = check_geom("fgx_spconv_out_dims", W, H, D, Kw, Kh, Kd, Sw, Sh, Sd, Pw, Ph, Pd, Dw, Dh, Dd, &g);
    if (rc != FGX_OK) return rc;
    FGX_CHECK_ARG(Wo && Ho && Do, "fgx_spconv_out_dims: null output");
    *Wo = g.Wo;
    *Ho = g.Ho;
    *Do = g.Do;
    return FGX_OK;
}

size_t fgx_spconv_out_coords_workspace_bytes(size_t n_in, int V, int key_bits) {
    if (V < 1 || (key_bits != 32 && key_bits != 64)) return 0;
    return coords_layout(n_in, V, key_bits).total;
}

int fgx_spconv_out_coords_keys(const int32_t* coords, size_t n_in, int B, int W, int H, int D, int Kw, int Kh, int Kd, int Sw,
                               int Sh, int Sd, int Pw, int Ph, int Pd, int Dw, int Dh, int Dd, int key_bits, void* workspace,
                               size_t workspace_bytes, uint64_t* count, fgx_stream_t stream) {
    ConvGeom g;
    int rc = check_geom("fgx_spconv_out_coords_keys", W, H, D, Kw, Kh, Kd, Sw, Sh, Sd, Pw, Ph, Pd, Dw, Dh, Dd, &g);
    if (rc != FGX_OK) return rc;
    FGX_CHECK_ARG(B > 0, "fgx_spconv_out_coords_keys: batch size must be positive");
    FGX_CHECK_ARG(key_bits == 32 || key_bits == 64, "fgx_spconv_out_coords_keys: key_bits must be 32 or 64, got %d", key_bits);
    FGX_CHECK_ARG(count != nullptr, "fgx_spconv_out_coords_keys: null count");
    hipStream_t s = (hipStream_t)stream;
    if (n_in == 0 || g.Wo <= 0 || g.Ho <= 0 || g.Do <= 0) {       // nothing can be reached
        fill_u32_kernel<<<1, kBlock, 0, s>>>((uint32_t*)count, 2, 0u);
        FGX_CHECK_LAUNCH("fgx_spconv_out_coords_keys(zero)");
        return FGX_OK;
    }
    // flattened (b, x, y, z) over the OUTPUT grid must leave room for the "unreachable" key one past the end
    const long double vol_ld = (long double)B * g.Wo * g.Ho * g.Do;
    FGX_CHECK_ARG(vol_ld < (key_bits == 32 ? 4294967295.0L : 18446744073709551615.0L),
                  "fgx_spconv_out_coords_keys: the output grid needs wider keys than %d bits", key_bits);
    const uint64_t vol = (uint64_t)B * (uint64_t)g.Wo * (uint64_t)g.Ho * (uint64_t)g.Do;
    FGX_CHECK_ARG(n_in * (size_t)g.V < ((size_t)1 << 40), "fgx_spconv_out_coords_keys: n*V too large");
    CoordsLayout L = coords_layout(n_in, g.V, key_bits);
    FGX_CHECK_ARG(coords && workspace, "fgx_spconv_out_coords_keys: null buffer");
    FGX_CHECK_ARG(((uintptr_t)coords & 15) == 0, "fgx_spconv_out_coords_keys: coords must be 16-byte aligned");
    FGX_CHECK_ARG(workspace_bytes >= L.total, "fgx_spconv_out_coords_keys: workspace of %zu bytes, need %zu", workspace_bytes, L.total);
    FGX_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fgx_spconv_out_coords_keys: workspace must be 256-byte aligned");
    char* ws = (char*)workspace;
    return key_bits == 32 ? out_coords_keys_impl<uint32_t>(coords, n_in, g, vol, ws, L, count, s)
                          : out_coords_keys_impl<uint64_t>(coords, n_in, g, vol, ws, L, count, s);
}

int fgx_spconv_out_coords_decode(const void* workspace, int key_bits, size_t count, int Wo, int Ho, int Do, int32_t* out_coords,
                                 fgx_stream_t stream) {
    FGX_CHECK_ARG(key_bits == 32 || key_bits == 64, "fgx_spconv_out_coords_decode: key_bits must be 32 or 64, got %d", key_bits);
    if (count == 0) return FGX_OK;
    FGX_CHECK_ARG(workspace && out_coords, "fgx_spconv_out_coords_decode: null buffer");
    FGX_CHECK_ARG(Wo > 0 && Ho > 0 && Do > 0, "fgx_spconv_out_coords_decode: output extents must be positive");
    FGX_CHECK_ARG(((uintptr_t)out_coords & 15) == 0, "fgx_spconv_out_coords_decode: out_coords must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    // the sorted unique keys sit at the start of the workspace
    if (key_bits == 32)
        decode_keys_kernel<uint32_t><<<cdiv(count, kBlock), kBlock, 0, s>>>((const uint32_t*)workspace, count, Wo, Ho, Do, out_coords);
    else
        decode_keys_kernel<uint64_t><<<cdiv(count, kBlock), kBlock, 0, s>>>((const uint64_t*)workspace, count, Wo, Ho, Do, out_coords);
    FGX_CHECK_LAUNCH("fgx_spconv_out_coords_decode");
    return FGX_OK;
}

int fgx_spconv_neighbor_map(const void* keys, int key_bits, const uint32_t* vals, size_t table_size, const int32_t* out_coords,
                            size_t n_out, size_t n_in, int W, int H, int D, int Kw, int Kh, int Kd, int Sw, int Sh, int Sd, int Pw,
                            int Ph, int Pd, int Dw, int Dh, int Dd, uint32_t* map_fwd, uint32_t* map_bwd, int32_t* gray,
                            int32_t* binary, fgx_stream_t stream) {
    ConvGeom g;
    int rc = check_geom("fgx_spconv_neighbor_map", W, H, D, Kw, Kh, Kd, Sw, Sh, Sd, Pw, Ph, Pd, Dw, Dh, Dd, &g);
    if (rc != FGX_OK) return rc;
    FGX_CHECK_ARG(key_bits == 32 || key_bits == 64, "fgx_spconv_neighbor_map: key_bits must be 32 or 64, got %d", key_bits);
    FGX_CHECK_ARG((gray == nullptr) == (binary == nullptr), "fgx_spconv_neighbor_map: gray and binary go together");
    FGX_CHECK_ARG(gray == nullptr || g.V <= 32, "fgx_spconv_neighbor_map: mask codes need a kernel volume <= 32, got %d", g.V);
    FGX_CHECK_ARG(n_out < 0xFFFFFFFFull && n_in < 0xFFFFFFFFull, "fgx_spconv_neighbor_map: row indices must fit below 2^32-1");
    hipStream_t s = (hipStream_t)stream;
    if (map_bwd != nullptr && n_in > 0) {
        const size_t cells = n_in * (size_t)g.V;
        unsigned grid = cdiv(cells, kBlock);
        if (grid > 65536u) grid = 65536u;
        fill_u32_kernel<<<grid, kBlock, 0, s>>>(map_bwd, cells, FGX_EMPTY32);
        FGX_CHECK_LAUNCH("fgx_spconv_neighbor_map(fill)");
    }
    if (n_out == 0) return FGX_OK;
    FGX_CHECK_ARG(out_coords && map_fwd, "fgx_spconv_neighbor_map: null buffer");
    FGX_CHECK_ARG(n_in == 0 || (table_size > 0 && keys && vals), "fgx_spconv_neighbor_map: null or empty table");
    FGX_CHECK_ARG(((uintptr_t)out_coords & 15) == 0, "fgx_spconv_neighbor_map: out_coords must be 16-byte aligned");
    FGX_CHECK_ARG(n_out * (size_t)g.V < ((size_t)1 << 40), "fgx_spconv_neighbor_map: n*V too large");
    if (n_in == 0) {       // no input voxel: every neighbor is absent
        const size_t cells = n_out * (size_t)g.V;
        unsigned grid = cdiv(cells, kBlock);
        if (grid > 65536u) grid = 65536u;
        fill_u32_kernel<<<grid, kBlock, 0, s>>>(map_fwd, cells, FGX_EMPTY32);
        FGX_CHECK_LAUNCH("fgx_spconv_neighbor_map(fill)");
        if (gray != nullptr) {
            fill_u32_kernel<<<cdiv(n_out, kBlock), kBlock, 0, s>>>((uint32_t*)gray, n_out, 0u);
            fill_u32_kernel<<<cdiv(n_out, kBlock), kBlock, 0, s>>>((uint32_t*)binary, n_out, 0u);
            FGX_CHECK_LAUNCH("fgx_spconv_neighbor_map(fill)");
        }
        return FGX_OK;
    }
    if (g.V <= 32) {
        const unsigned grid = cdiv(n_out * 32, kBlock);
        if (key_bits == 32)
            spconv_map_halfwave_kernel<uint32_t><<<grid, kBlock, 0, s>>>((const uint32_t*)keys, vals, table_size, out_coords, n_out, g,
                                                                        map_fwd, map_bwd, gray, binary);
        else
            spconv_map_halfwave_kernel<uint64_t><<<grid, kBlock, 0, s>>>((const uint64_t*)keys, vals, table_size, out_coords, n_out, g,
                                                                        map_fwd, map_bwd, gray, binary);
    } else {
        const unsigned grid = cdiv(n_out * (size_t)g.V, kBlock);
        if (key_bits == 32)
            spconv_map_flat_kernel<uint32_t><<<grid, kBlock, 0, s>>>((const uint32_t*)keys, vals, table_size, out_coords, n_out, g,
                                                                    map_fwd, map_bwd);
        else
            spconv_map_flat_kernel<uint64_t><<<grid, kBlock, 0, s>>>((const uint64_t*)keys, vals, table_size, out_coords, n_out, g,
                                                                    map_fwd, map_bwd);
    }
    FGX_CHECK_LAUNCH("fgx_spconv_neighbor_map");
    return FGX_OK;
}

}  // extern "C"
