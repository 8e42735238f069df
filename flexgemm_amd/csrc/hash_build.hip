// Open-addressing hash table and the submanifold neighbor-map builder for gfx950.
//
// Table semantics follow the reference (flex_gemm/kernels/cuda/hash/hash.cuh:5-129): Murmur3
// finaliser modulo the table size, linear probing with wrap-around, all-ones key = empty,
// compare-and-swap insert, lock-free lookup.
//
// The neighbor-map kernel is laid out for 64-wide wavefronts instead of the reference's
// (V/2+1)-threads-per-voxel mirror scheme (subm_neighbor_map.cu:33-83): one half-wave (32 lanes)
// owns one voxel, lane v < V probes offset v, the 4*V-byte row is written with one coalesced
// store, and the half-wave ballot of "found" IS the validity mask, so the Gray/binary codes come
// out of the same pass without re-reading the map.
#include <stdarg.h>
#include <limits>

#include "fgx_common.h"
#include "hash_device.h"

namespace fgx {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

static fgx_phase_hook_t g_phase_hook = nullptr;

void phase_mark(const char* name, hipStream_t s) {
    if (g_phase_hook) g_phase_hook(name, (fgx_stream_t)s);
}

namespace {

constexpr int kBlock = 256;

template <typename K>
__global__ void __launch_bounds__(kBlock) fill_keys_kernel(K* keys, size_t table) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    size_t stride = (size_t)gridDim.x * kBlock;
    for (; i < table; i += stride) keys[i] = std::numeric_limits<K>::max();
}

template <typename K, typename Val>
__global__ void __launch_bounds__(kBlock) insert_kernel(K* keys, Val* vals, size_t table, const K* in_keys,
                                                        const Val* in_vals, size_t m) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < m) probe_insert(keys, vals, in_keys[i], in_vals[i], table);
}

template <typename K, typename Val>
__global__ void __launch_bounds__(kBlock) lookup_kernel(const K* keys, const Val* vals, size_t table,
                                                        const K* in_keys, Val* out_vals, size_t m) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < m) out_vals[i] = probe_lookup(keys, vals, in_keys[i], table);
}

// in_vals == nullptr: the value is the row index.
template <typename K, typename Val>
__global__ void __launch_bounds__(kBlock) insert_3d_kernel(K* keys, Val* vals, size_t table, const int32_t* coords,
                                                           const Val* in_vals, size_t m, int W, int H, int D) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < m) {
        int4 c = reinterpret_cast<const int4*>(coords)[i];
        K key = (K)flat_key(c.x, c.y, c.z, c.w, W, H, D);
        Val val = in_vals ? in_vals[i] : (Val)i;
        probe_insert(keys, vals, key, val, table);
    }
}

template <typename K, typename Val>
__global__ void __launch_bounds__(kBlock) lookup_3d_kernel(const K* keys, const Val* vals, size_t table,
                                                           const int32_t* coords, Val* out_vals, size_t m,
                                                           int W, int H, int D) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < m) {
        int4 c = reinterpret_cast<const int4*>(coords)[i];
        Val r = std::numeric_limits<Val>::max();
        if (c.y >= 0 && c.y < W && c.z >= 0 && c.z < H && c.w >= 0 && c.w < D)
            r = probe_lookup(keys, vals, (K)flat_key(c.x, c.y, c.z, c.w, W, H, D), table);
        out_vals[i] = r;
    }
}

__device__ __forceinline__ uint32_t gray_to_binary(uint32_t g) {
    uint32_t b = g;
    b ^= b >> 1;
    b ^= b >> 2;
    b ^= b >> 4;
    b ^= b >> 8;
    b ^= b >> 16;
    return b;
}

// Half-wave per voxel, V <= 32.  Lane v probes offset v (x-major flattening); the centre lane is
// the voxel itself.
template <typename K>
__global__ void __launch_bounds__(kBlock) neighbor_map_halfwave_kernel(
    const K* __restrict__ keys, const uint32_t* __restrict__ vals, size_t table,
    const int32_t* __restrict__ coords, size_t n, int W, int H, int D, int V, int Kw, int Kh, int Kd,
    int Dw, int Dh, int Dd, uint32_t* __restrict__ out_map, int32_t* __restrict__ gray,
    int32_t* __restrict__ binary) {
    const size_t voxel = ((size_t)blockIdx.x * kBlock + threadIdx.x) >> 5;
    const int v = threadIdx.x & 31;
    const bool active = voxel < n && v < V;
    uint32_t value = FGX_EMPTY32;
    if (active) {
        int4 c = reinterpret_cast<const int4*>(coords)[voxel];
        if (v == V / 2) {
            value = (uint32_t)voxel;
        } else {
            int kx = c.y + (v / (Kh * Kd) - Kw / 2) * Dw;
            int ky = c.z + (v / Kd % Kh - Kh / 2) * Dh;
            int kz = c.w + (v % Kd - Kd / 2) * Dd;
            if (kx >= 0 && kx < W && ky >= 0 && ky < H && kz >= 0 && kz < D)
                value = probe_lookup(keys, vals, (K)flat_key(c.x, kx, ky, kz, W, H, D), table);
        }
        out_map[voxel * (size_t)V + v] = value;
    }
    if (gray != nullptr) {
        unsigned long long found = __ballot(active && value != FGX_EMPTY32);
        uint32_t g = (uint32_t)(found >> (threadIdx.x & 32));
        if (v == 0 && voxel < n) {
            gray[voxel] = (int32_t)g;
            binary[voxel] = (int32_t)gray_to_binary(g);
        }
    }
}

// Any V: one thread per (voxel, offset).
template <typename K>
__global__ void __launch_bounds__(kBlock) neighbor_map_flat_kernel(
    const K* __restrict__ keys, const uint32_t* __restrict__ vals, size_t table,
    const int32_t* __restrict__ coords, size_t n, int W, int H, int D, int V, int Kw, int Kh, int Kd,
    int Dw, int Dh, int Dd, uint32_t* __restrict__ out_map) {
    const size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= n * (size_t)V) return;
    const size_t voxel = t / V;
    const int v = (int)(t % V);
    int4 c = reinterpret_cast<const int4*>(coords)[voxel];
    uint32_t value = FGX_EMPTY32;
    if (v == V / 2) {
        value = (uint32_t)voxel;
    } else {
        int kx = c.y + (v / (Kh * Kd) - Kw / 2) * Dw;
        int ky = c.z + (v / Kd % Kh - Kh / 2) * Dh;
        int kz = c.w + (v % Kd - Kd / 2) * Dd;
        if (kx >= 0 && kx < W && ky >= 0 && ky < H && kz >= 0 && kz < D)
            value = probe_lookup(keys, vals, (K)flat_key(c.x, kx, ky, kz, W, H, D), table);
    }
    out_map[t] = value;
}

__global__ void __launch_bounds__(kBlock) mask_codes_kernel(const uint32_t* __restrict__ map, size_t n, int V,
                                                            int32_t* __restrict__ gray,
                                                            int32_t* __restrict__ binary) {
    // half-wave per voxel: coalesced row read, ballot = mask
    const size_t voxel = ((size_t)blockIdx.x * kBlock + threadIdx.x) >> 5;
    const int v = threadIdx.x & 31;
    bool present = false;
    if (voxel < n && v < V) present = map[voxel * (size_t)V + v] != FGX_EMPTY32;
    unsigned long long found = __ballot(present);
    uint32_t g = (uint32_t)(found >> (threadIdx.x & 32));
    if (v == 0 && voxel < n) {
        gray[voxel] = (int32_t)g;
        binary[voxel] = (int32_t)gray_to_binary(g);
    }
}

bool bits_ok(int b) { return b == 32 || b == 64; }

template <typename F>
int dispatch_kv(int key_bits, int val_bits, F&& f) {
    if (key_bits == 32 && val_bits == 32) return f((uint32_t*)nullptr, (uint32_t*)nullptr);
    if (key_bits == 32 && val_bits == 64) return f((uint32_t*)nullptr, (uint64_t*)nullptr);
    if (key_bits == 64 && val_bits == 32) return f((uint64_t*)nullptr, (uint32_t*)nullptr);
    return f((uint64_t*)nullptr, (uint64_t*)nullptr);
}

}  // namespace
}  // namespace fgx

using namespace fgx;

extern "C" {

int fgx_abi_version(void) { return 2; }

void fgx_set_phase_hook(fgx_phase_hook_t hook) { fgx::g_phase_hook = hook; }

const char* fgx_last_error(void) { return fgx::g_error; }

int fgx_hash_init(void* keys, int key_bits, size_t table_size, fgx_stream_t stream) {
    FGX_CHECK_ARG(bits_ok(key_bits), "fgx_hash_init: key_bits must be 32 or 64, got %d", key_bits);
    if (table_size == 0) return FGX_OK;
    FGX_CHECK_ARG(keys != nullptr, "fgx_hash_init: null key table");
    hipStream_t s = (hipStream_t)stream;
    unsigned grid = cdiv(table_size, kBlock);
    if (grid > 65536u) grid = 65536u;
    if (key_bits == 32) fill_keys_kernel<uint32_t><<<grid, kBlock, 0, s>>>((uint32_t*)keys, table_size);
    else fill_keys_kernel<uint64_t><<<grid, kBlock, 0, s>>>((uint64_t*)keys, table_size);
    FGX_CHECK_LAUNCH("fgx_hash_init");
    return FGX_OK;
}

int fgx_hash_insert(void* keys, int key_bits, void* vals, int val_bits, size_t table_size, const void* in_keys,
                    const void* in_vals, size_t m, fgx_stream_t stream) {
    FGX_CHECK_ARG(bits_ok(key_bits) && bits_ok(val_bits), "fgx_hash_insert: unsupported key/value width %d/%d", key_bits, val_bits);
    if (m == 0) return FGX_OK;
    FGX_CHECK_ARG(table_size > 0 && keys && vals && in_keys && in_vals, "fgx_hash_insert: null buffer or empty table");
    hipStream_t s = (hipStream_t)stream;
    return dispatch_kv(key_bits, val_bits, [&](auto* kt, auto* vt) {
        using K = std::remove_pointer_t<decltype(kt)>;
        using Vv = std::remove_pointer_t<decltype(vt)>;
        insert_kernel<K, Vv><<<cdiv(m, kBlock), kBlock, 0, s>>>((K*)keys, (Vv*)vals, table_size, (const K*)in_keys,
                                                                (const Vv*)in_vals, m);
        FGX_CHECK_LAUNCH("fgx_hash_insert");
        return FGX_OK;
    });
}

int fgx_hash_lookup(const void* keys, int key_bits, const void* vals, int val_bits, size_t table_size,
                    const void* in_keys, void* out_vals, size_t m, fgx_stream_t stream) {
    FGX_CHECK_ARG(bits_ok(key_bits) && bits_ok(val_bits), "fgx_hash_lookup: unsupported key/value width %d/%d", key_bits, val_bits);
    if (m == 0) return FGX_OK;
    FGX_CHECK_ARG(table_size > 0 && keys && vals && in_keys && out_vals, "fgx_hash_lookup: null buffer or empty table");
    hipStream_t s = (hipStream_t)stream;
    return dispatch_kv(key_bits, val_bits, [&](auto* kt, auto* vt) {
        using K = std::remove_pointer_t<decltype(kt)>;
        using Vv = std::remove_pointer_t<decltype(vt)>;
        lookup_kernel<K, Vv><<<cdiv(m, kBlock), kBlock, 0, s>>>((const K*)keys, (const Vv*)vals, table_size,
                                                                (const K*)in_keys, (Vv*)out_vals, m);
        FGX_CHECK_LAUNCH("fgx_hash_lookup");
        return FGX_OK;
    });
}

int fgx_hash_insert_3d(void* keys, int key_bits, void* vals, int val_bits, size_t table_size, const int32_t* coords,
                       const void* in_vals, size_t m, int W, int H, int D, fgx_stream_t stream) {
    FGX_CHECK_ARG(bits_ok(key_bits) && bits_ok(val_bits), "fgx_hash_insert_3d: unsupported key/value width %d/%d", key_bits, val_bits);
    if (m == 0) return FGX_OK;
    FGX_CHECK_ARG(table_size > 0 && keys && vals && coords && in_vals, "fgx_hash_insert_3d: null buffer or empty table");
    FGX_CHECK_ARG(((uintptr_t)coords & 15) == 0, "fgx_hash_insert_3d: coords must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    return dispatch_kv(key_bits, val_bits, [&](auto* kt, auto* vt) {
        using K = std::remove_pointer_t<decltype(kt)>;
        using Vv = std::remove_pointer_t<decltype(vt)>;
        insert_3d_kernel<K, Vv><<<cdiv(m, kBlock), kBlock, 0, s>>>((K*)keys, (Vv*)vals, table_size, coords,
                                                                   (const Vv*)in_vals, m, W, H, D);
        FGX_CHECK_LAUNCH("fgx_hash_insert_3d");
        return FGX_OK;
    });
}

int fgx_hash_insert_3d_idx_as_val(void* keys, int key_bits, void* vals, int val_bits, size_t table_size,
                                  const int32_t* coords, size_t n, int W, int H, int D, fgx_stream_t stream) {
    FGX_CHECK_ARG(bits_ok(key_bits) && bits_ok(val_bits), "fgx_hash_insert_3d_idx_as_val: unsupported key/value width %d/%d", key_bits, val_bits);
    if (n == 0) return FGX_OK;
    FGX_CHECK_ARG(table_size > 0 && keys && vals && coords, "fgx_hash_insert_3d_idx_as_val: null buffer or empty table");
    FGX_CHECK_ARG(((uintptr_t)coords & 15) == 0, "fgx_hash_insert_3d_idx_as_val: coords must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    return dispatch_kv(key_bits, val_bits, [&](auto* kt, auto* vt) {
        using K = std::remove_pointer_t<decltype(kt)>;
        using Vv = std::remove_pointer_t<decltype(vt)>;
        insert_3d_kernel<K, Vv><<<cdiv(n, kBlock), kBlock, 0, s>>>((K*)keys, (Vv*)vals, table_size, coords,
                                                                   (const Vv*)nullptr, n, W, H, D);
        FGX_CHECK_LAUNCH("fgx_hash_insert_3d_idx_as_val");
        return FGX_OK;
    });
}

int fgx_hash_lookup_3d(const void* keys, int key_bits, const void* vals, int val_bits, size_t table_size,
                       const int32_t* coords, void* out_vals, size_t m, int W, int H, int D, fgx_stream_t stream) {
    FGX_CHECK_ARG(bits_ok(key_bits) && bits_ok(val_bits), "fgx_hash_lookup_3d: unsupported key/value width %d/%d", key_bits, val_bits);
    if (m == 0) return FGX_OK;
    FGX_CHECK_ARG(table_size > 0 && keys && vals && coords && out_vals, "fgx_hash_lookup_3d: null buffer or empty table");
    FGX_CHECK_ARG(((uintptr_t)coords & 15) == 0, "fgx_hash_lookup_3d: coords must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    return dispatch_kv(key_bits, val_bits, [&](auto* kt, auto* vt) {
        using K = std::remove_pointer_t<decltype(kt)>;
        using Vv = std::remove_pointer_t<decltype(vt)>;
        lookup_3d_kernel<K, Vv><<<cdiv(m, kBlock), kBlock, 0, s>>>((const K*)keys, (const Vv*)vals, table_size, coords,
                                                                   (Vv*)out_vals, m, W, H, D);
        FGX_CHECK_LAUNCH("fgx_hash_lookup_3d");
        return FGX_OK;
    });
}

int fgx_subm_neighbor_map(void* keys, int key_bits, uint32_t* vals, size_t table_size, const int32_t* coords, size_t n,
                          int W, int H, int D, int Kw, int Kh, int Kd, int Dw, int Dh, int Dd, uint32_t* out_map,
                          int32_t* gray, int32_t* binary, fgx_stream_t stream) {
    FGX_CHECK_ARG(bits_ok(key_bits), "fgx_subm_neighbor_map: key_bits must be 32 or 64, got %d", key_bits);
    FGX_CHECK_ARG(Kw > 0 && Kh > 0 && Kd > 0 && (Kw & 1) && (Kh & 1) && (Kd & 1),
                  "fgx_subm_neighbor_map: kernel sizes must be odd and positive, got (%d,%d,%d)", Kw, Kh, Kd);
    FGX_CHECK_ARG(W > 0 && H > 0 && D > 0, "fgx_subm_neighbor_map: grid extents must be positive");
    FGX_CHECK_ARG((gray == nullptr) == (binary == nullptr), "fgx_subm_neighbor_map: gray and binary go together");
    const long long Vll = (long long)Kw * Kh * Kd;
    FGX_CHECK_ARG(Vll <= 1 << 20, "fgx_subm_neighbor_map: kernel volume too large");
    const int V = (int)Vll;
    FGX_CHECK_ARG(gray == nullptr || V <= 32, "fgx_subm_neighbor_map: mask codes need a kernel volume <= 32, got %d", V);
    FGX_CHECK_ARG(n < 0xFFFFFFFFull, "fgx_subm_neighbor_map: row indices must fit below 2^32-1");
    if (n == 0) return FGX_OK;
    FGX_CHECK_ARG(table_size >= n, "fgx_subm_neighbor_map: table of %zu slots cannot hold %zu voxels", table_size, n);
    FGX_CHECK_ARG(keys && vals && coords && out_map, "fgx_subm_neighbor_map: null buffer");
    FGX_CHECK_ARG(((uintptr_t)coords & 15) == 0, "fgx_subm_neighbor_map: coords must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    PhaseEnd phases{s};
    phase_mark("hash insert", s);
    int rc = fgx_hash_insert_3d_idx_as_val(keys, key_bits, vals, 32, table_size, coords, n, W, H, D, stream);
    if (rc != FGX_OK) return rc;
    phase_mark("hash probe", s);
    if (V <= 32) {
        unsigned grid = cdiv(n * 32, kBlock);
        if (key_bits == 32)
            neighbor_map_halfwave_kernel<uint32_t><<<grid, kBlock, 0, s>>>((const uint32_t*)keys, vals, table_size, coords, n, W, H, D, V,
                                                                          Kw, Kh, Kd, Dw, Dh, Dd, out_map, gray, binary);
        else
            neighbor_map_halfwave_kernel<uint64_t><<<grid, kBlock, 0, s>>>((const uint64_t*)keys, vals, table_size, coords, n, W, H, D, V,
                                                                          Kw, Kh, Kd, Dw, Dh, Dd, out_map, gray, binary);
    } else {
        FGX_CHECK_ARG(n * (size_t)V < ((size_t)1 << 40), "fgx_subm_neighbor_map: n*V too large");
        unsigned grid = cdiv(n * (size_t)V, kBlock);
        if (key_bits == 32)
            neighbor_map_flat_kernel<uint32_t><<<grid, kBlock, 0, s>>>((const uint32_t*)keys, vals, table_size, coords, n, W, H, D, V, Kw,
                                                                      Kh, Kd, Dw, Dh, Dd, out_map);
        else
            neighbor_map_flat_kernel<uint64_t><<<grid, kBlock, 0, s>>>((const uint64_t*)keys, vals, table_size, coords, n, W, H, D, V, Kw,
                                                                      Kh, Kd, Dw, Dh, Dd, out_map);
    }
    FGX_CHECK_LAUNCH("fgx_subm_neighbor_map");
    return FGX_OK;
}

int fgx_mask_codes(const uint32_t* map, size_t n, int V, int32_t* gray, int32_t* binary, fgx_stream_t stream) {
    FGX_CHECK_ARG(V >= 1 && V <= 32, "fgx_mask_codes: kernel volume must be in [1, 32], got %d", V);
    if (n == 0) return FGX_OK;
    FGX_CHECK_ARG(map && gray && binary, "fgx_mask_codes: null buffer");
    mask_codes_kernel<<<cdiv(n * 32, kBlock), kBlock, 0, (hipStream_t)stream>>>(map, n, V, gray, binary);
    FGX_CHECK_LAUNCH("fgx_mask_codes");
    return FGX_OK;
}

}  // extern "C"
