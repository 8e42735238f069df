// Submanifold neighbor map by sorting and merging instead of hashing, for gfx950.
//
// The hash builder (hash_build.hip, the reference's scheme: flex_gemm/kernels/cuda/spconv/subm_neighbor_map.cu:33-162)
// answers every (voxel, offset) question with a probe at a pseudo-random table slot: V - 1 dependent cache-line
// fetches per voxel from a table several times the size of an L2.  The result -- map[n, v] = row of the voxel at
// coords[n] + delta_v -- does not depend on how it is found, and the flattened key ((b*W + x)*H + y)*D + z orders the
// voxels so that the answers to neighboring questions sit next to each other:
//
//   * sort (key, row) pairs once (radix sort over the bits a key can have);
//   * the voxels of one workgroup are 256 consecutive sorted entries; for a fixed (dx, dy) their neighbors' keys are the
//     same keys shifted by a constant, so they all fall into ONE contiguous window of the sorted array, whose ends two
//     binary searches find;
//   * the window is read once, coalesced, into LDS, and every lane finds its Kd neighbors along z there.
//
// All traffic is sequential except the final row-wise scatter of the 4*V-byte map rows back to input order.
#include <cstring>
#include <string.h>

#include <rocprim/rocprim.hpp>

#include "fgx_common.h"

namespace fgx {
namespace {

constexpr int kGroup = 256;      // sorted voxels per workgroup
constexpr int kWindow = 768;     // window entries held in LDS per (dx, dy) row; larger windows are searched in place
constexpr int kMaxRows = 128;    // Kw * Kh
constexpr int kStageV = 32;      // kernel volumes up to this many positions have their map rows staged in LDS

struct SubmGeom {
    int W, H, D;
    int Kw, Kh, Kd, V;
    int Dw, Dh, Dd;
};

template <typename K>
__global__ void __launch_bounds__(256) flat_keys_kernel(const int32_t* __restrict__ coords, size_t n, int W, int H, int D,
                                                        K* __restrict__ keys, uint32_t* __restrict__ rows) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int4 c = reinterpret_cast<const int4*>(coords)[i];
    keys[i] = (K)((((uint64_t)(uint32_t)c.x * (uint64_t)W + (uint64_t)c.y) * (uint64_t)H + (uint64_t)c.z) * (uint64_t)D + (uint64_t)c.w);
    rows[i] = (uint32_t)i;
}

// first position in a[lo, hi) whose key is >= t (hi if none)
template <typename K>
__device__ __forceinline__ size_t lower_bound_at(const K* a, size_t lo, size_t hi, K t) {
    while (lo < hi) {
        const size_t mid = lo + ((hi - lo) >> 1);
        if (a[mid] < t) lo = mid + 1;
        else hi = mid;
    }
    return lo;
}

__device__ __forceinline__ uint32_t gray_decode(uint32_t g) {
    g ^= g >> 16;
    g ^= g >> 8;
    g ^= g >> 4;
    g ^= g >> 2;
    g ^= g >> 1;
    return g;
}

// bounds[(group * R + r) * 2 + {0, 1}] = [first, one past last) position of the window of sorted keys in which the
// (dx, dy) = r neighbors of the group's voxels lie: the group's own key range shifted by the row's constant and
// widened by the reach along z.  One thread per bound: the searches of all groups overlap.
template <typename K>
__global__ void __launch_bounds__(256) window_bounds_kernel(const K* __restrict__ skeys, size_t n, unsigned long long vol,
                                                            SubmGeom g, unsigned groups, uint32_t* __restrict__ bounds) {
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int R = g.Kw * g.Kh;
    if (t >= (size_t)groups * R * 2) return;
    const size_t grp = t / (2 * R);
    const int r = (int)(t % (2 * R)) >> 1;
    const size_t p0 = grp * kGroup;
    const size_t cnt = n - p0 < (size_t)kGroup ? n - p0 : (size_t)kGroup;
    const long long HD = (long long)g.H * g.D;
    const long long half_z = (long long)(g.Kd / 2) * g.Dd;
    const long long off = (long long)(r / g.Kh - g.Kw / 2) * g.Dw * HD + (long long)(r % g.Kh - g.Kh / 2) * g.Dh * g.D;
    // 64-bit keys stay below 2^63 (the caller checks), so signed arithmetic cannot wrap
    const long long lo_t = (long long)skeys[p0] + off - half_z, hi_t = (long long)skeys[p0 + cnt - 1] + off + half_z;
    // keys lie in [0, vol): targets outside need no search (and must not be narrowed to K)
    size_t pos;
    if ((t & 1) == 0) pos = hi_t < 0 ? 0 : (lo_t >= (long long)vol ? n : lower_bound_at<K>(skeys, 0, n, (K)(lo_t < 0 ? 0 : lo_t)));
    else pos = hi_t < 0 ? 0 : (hi_t + 1 >= (long long)vol ? n : lower_bound_at<K>(skeys, 0, n, (K)(hi_t + 1)));   // first key > hi_t
    bounds[t] = (uint32_t)pos;
}

template <typename K>
__global__ void __launch_bounds__(kGroup) merge_neighbor_kernel(const K* __restrict__ skeys, const uint32_t* __restrict__ srows,
                                                                const uint32_t* __restrict__ bounds, size_t n, SubmGeom g,
                                                                uint32_t* __restrict__ out_map,
                                                                int32_t* __restrict__ gray, int32_t* __restrict__ binary) {
    constexpr int kPer = kWindow / kGroup;      // window entries a lane carries from memory to LDS
    __shared__ K wkeys[kWindow];
    __shared__ uint32_t wrows[kWindow];
    __shared__ uint32_t win_lo[kMaxRows], win_hi[kMaxRows];
    // map rows of the group, so that each leaves as one contiguous 4*V-byte store instead of V scattered words
    // (pitch V + 1 words: lanes of a wavefront write the same column of consecutive rows)
    __shared__ uint32_t out_rows[kGroup * (kStageV + 1)];
    __shared__ uint32_t out_dst[kGroup];
    const bool stage_out = g.V <= kStageV;
    const size_t p0 = (size_t)blockIdx.x * kGroup;
    const int cnt = (int)(n - p0 < (size_t)kGroup ? n - p0 : (size_t)kGroup);
    const int tid = threadIdx.x;
    const bool live = tid < cnt;
    const int R = g.Kw * g.Kh;
    const long long HD = (long long)g.H * g.D;

    for (int j = tid; j < R; j += kGroup) {
        win_lo[j] = bounds[((size_t)blockIdx.x * R + j) * 2];
        win_hi[j] = bounds[((size_t)blockIdx.x * R + j) * 2 + 1];
    }
    K key = 0;
    uint32_t me = 0;
    int x = 0, y = 0, z = 0;
    if (live) {
        key = skeys[p0 + tid];
        me = srows[p0 + tid];
        uint64_t t = (uint64_t)key;
        z = (int)(t % (uint64_t)g.D);
        t /= (uint64_t)g.D;
        y = (int)(t % (uint64_t)g.H);
        t /= (uint64_t)g.H;
        x = (int)(t % (uint64_t)g.W);
    }
    __syncthreads();

    // The windows of the next kAhead (dx, dy) rows travel from memory to registers together, so their latencies overlap;
    // each is then put into LDS and searched in turn.
    constexpr int kAhead = 9;
    K pk[kAhead][kPer];
    uint32_t pr[kAhead][kPer];
    uint32_t mask = 0;
    for (int r0 = 0; r0 < R; r0 += kAhead) {
#pragma unroll
        for (int a = 0; a < kAhead; ++a) {
            const int r = r0 + a;
            if (r >= R) break;
            const size_t lo = win_lo[r], hi = win_hi[r];
            const size_t w = hi > lo ? hi - lo : 0;
            if (w > (size_t)kWindow) continue;          // searched in place
#pragma unroll
            for (int i = 0; i < kPer; ++i) {
                const size_t j = (size_t)tid + (size_t)i * kGroup;
                if (j < w) {
                    pk[a][i] = skeys[lo + j];
                    pr[a][i] = srows[lo + j];
                }
            }
        }
#pragma unroll
        for (int a = 0; a < kAhead; ++a) {
            const int r = r0 + a;
            if (r >= R) break;
            const size_t lo = win_lo[r], hi = win_hi[r];
            const size_t w = hi > lo ? hi - lo : 0;
            const bool staged = w <= (size_t)kWindow;
            if (staged) {
#pragma unroll
                for (int i = 0; i < kPer; ++i) {
                    const size_t j = (size_t)tid + (size_t)i * kGroup;
                    if (j < w) {
                        wkeys[j] = pk[a][i];
                        wrows[j] = pr[a][i];
                    }
                }
            }
            __syncthreads();
            if (live) {
                const int kx = r / g.Kh, ky = r % g.Kh;
                const int x2 = x + (kx - g.Kw / 2) * g.Dw, y2 = y + (ky - g.Kh / 2) * g.Dh;
                const bool row_in = x2 >= 0 && x2 < g.W && y2 >= 0 && y2 < g.H;
                const long long off = (long long)(kx - g.Kw / 2) * g.Dw * HD + (long long)(ky - g.Kh / 2) * g.Dh * g.D;
                uint32_t* out_row = stage_out ? out_rows + tid * (kStageV + 1) + r * g.Kd
                                              : out_map + (size_t)me * g.V + (size_t)r * g.Kd;
                // the Kd targets of a row ascend by Dd: one binary search for the first, then a short walk to each next one
                unsigned pos = 0;
                bool searched = false;
                const unsigned wn = (unsigned)w;
                for (int kz = 0; kz < g.Kd; ++kz) {
                    const int dz = (kz - g.Kd / 2) * g.Dd;
                    const int z2 = z + dz;
                    uint32_t value = FGX_EMPTY32;
                    if (row_in && z2 >= 0 && z2 < g.D && w > 0) {
                        const K target = (K)((long long)key + off + dz);
                        if (staged) {
                            if (!searched) {
                                unsigned a = 0, b = wn;
                                while (a < b) {
                                    const unsigned mid = (a + b) >> 1;
                                    if (wkeys[mid] < target) a = mid + 1;
                                    else b = mid;
                                }
                                pos = a;
                                searched = true;
                            } else {
                                while (pos < wn && wkeys[pos] < target) ++pos;
                            }
                            if (pos < wn && wkeys[pos] == target) value = wrows[pos];
                        } else {
                            const size_t q = lower_bound_at<K>(skeys, lo, hi, target);
                            if (q < hi && skeys[q] == target) value = srows[q];
                        }
                    }
                    out_row[kz] = value;
                    const int v = r * g.Kd + kz;
                    if (v < 32 && value != FGX_EMPTY32) mask |= 1u << v;
                }
            }
            __syncthreads();       // the window is overwritten by the next row
        }
    }
    if (live && gray != nullptr) {
        gray[me] = (int32_t)mask;
        binary[me] = (int32_t)gray_decode(mask);
    }
    if (stage_out) {
        out_dst[tid] = me;
        __syncthreads();
        // one half-wavefront per row: lane v writes word v of the row
        const int lane32 = tid & 31;
        for (int row = tid >> 5; row < cnt; row += kGroup / 32)
            if (lane32 < g.V) out_map[(size_t)out_dst[row] * g.V + lane32] = out_rows[row * (kStageV + 1) + lane32];
    }
}

struct SortedLayout {
    size_t keys_in, keys_out, rows_in, rows_out, bounds, temp, temp_bytes, total;
};

template <typename K>
size_t pair_sort_temp_bytes(size_t n) {
    size_t bytes = 0;
    (void)rocprim::radix_sort_pairs(nullptr, bytes, (const K*)nullptr, (K*)nullptr, (const uint32_t*)nullptr, (uint32_t*)nullptr,
                                    n ? n : 1, 0u, (unsigned)(8 * sizeof(K)), (hipStream_t)0);
    return bytes;
}

SortedLayout sorted_layout(size_t n, int key_bits, int rows_xy) {
    SortedLayout L{};
    const size_t nn = n ? n : 1, es = key_bits / 8;
    size_t off = 0;
    L.keys_in = off;
    off = align_up(off + nn * es, 256);
    L.keys_out = off;
    off = align_up(off + nn * es, 256);
    L.rows_in = off;
    off = align_up(off + nn * 4, 256);
    L.rows_out = off;
    off = align_up(off + nn * 4, 256);
    L.bounds = off;
    off = align_up(off + (size_t)cdiv(nn, kGroup) * rows_xy * 2 * sizeof(uint32_t), 256);
    L.temp = off;
    L.temp_bytes = key_bits == 32 ? pair_sort_temp_bytes<uint32_t>(n) : pair_sort_temp_bytes<uint64_t>(n);
    L.total = off + align_up(L.temp_bytes, 256);
    return L;
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
int build_sorted(const int32_t* coords, size_t n, uint64_t vol, const SubmGeom& g, char* ws, const SortedLayout& L,
                 uint32_t* out_map, int32_t* gray, int32_t* binary, hipStream_t s) {
    K* keys_in = (K*)(ws + L.keys_in);
    K* keys_out = (K*)(ws + L.keys_out);
    uint32_t* rows_in = (uint32_t*)(ws + L.rows_in);
    uint32_t* rows_out = (uint32_t*)(ws + L.rows_out);
    flat_keys_kernel<K><<<cdiv(n, 256), 256, 0, s>>>(coords, n, g.W, g.H, g.D, keys_in, rows_in);
    FGX_CHECK_LAUNCH("fgx_subm_neighbor_map_sorted(keys)");
    size_t temp_bytes = L.temp_bytes;
    unsigned end_bit = bit_length(vol - 1);
    if (end_bit == 0) end_bit = 1;
    FGX_CHECK_HIP(rocprim::radix_sort_pairs(ws + L.temp, temp_bytes, (const K*)keys_in, keys_out, (const uint32_t*)rows_in, rows_out,
                                            n, 0u, end_bit, s));
    const unsigned groups = cdiv(n, kGroup);
    uint32_t* bounds = (uint32_t*)(ws + L.bounds);
    window_bounds_kernel<K><<<cdiv((size_t)groups * g.Kw * g.Kh * 2, 256), 256, 0, s>>>(keys_out, n, (unsigned long long)vol, g, groups, bounds);
    FGX_CHECK_LAUNCH("fgx_subm_neighbor_map_sorted(bounds)");
    merge_neighbor_kernel<K><<<groups, kGroup, 0, s>>>(keys_out, rows_out, bounds, n, g, out_map, gray, binary);
    FGX_CHECK_LAUNCH("fgx_subm_neighbor_map_sorted");
    return FGX_OK;
}

}  // namespace
}  // namespace fgx

using namespace fgx;

extern "C" {

size_t fgx_subm_neighbor_map_sorted_workspace_bytes(size_t n, int key_bits, int Kw, int Kh) {
    if ((key_bits != 32 && key_bits != 64) || Kw < 1 || Kh < 1 || Kw * Kh > kMaxRows) return 0;
    return sorted_layout(n, key_bits, Kw * Kh).total;
}

int fgx_subm_neighbor_map_sorted(const int32_t* coords, size_t n, int B, int W, int H, int D, int Kw, int Kh, int Kd, int Dw,
                                 int Dh, int Dd, int key_bits, void* workspace, size_t workspace_bytes, uint32_t* out_map,
                                 int32_t* gray, int32_t* binary, fgx_stream_t stream) {
    FGX_CHECK_ARG(key_bits == 32 || key_bits == 64, "fgx_subm_neighbor_map_sorted: key_bits must be 32 or 64, got %d", key_bits);
    FGX_CHECK_ARG(Kw > 0 && Kh > 0 && Kd > 0 && (Kw & 1) && (Kh & 1) && (Kd & 1),
                  "fgx_subm_neighbor_map_sorted: kernel sizes must be odd and positive, got (%d,%d,%d)", Kw, Kh, Kd);
    FGX_CHECK_ARG(B > 0 && W > 0 && H > 0 && D > 0, "fgx_subm_neighbor_map_sorted: grid extents must be positive");
    FGX_CHECK_ARG(Dw > 0 && Dh > 0 && Dd > 0, "fgx_subm_neighbor_map_sorted: dilations must be positive");
    FGX_CHECK_ARG((gray == nullptr) == (binary == nullptr), "fgx_subm_neighbor_map_sorted: gray and binary go together");
    FGX_CHECK_ARG(Kw * Kh <= kMaxRows && (long long)Kw * Kh * Kd <= 1 << 20, "fgx_subm_neighbor_map_sorted: kernel too large");
    const int V = Kw * Kh * Kd;
    FGX_CHECK_ARG(gray == nullptr || V <= 32, "fgx_subm_neighbor_map_sorted: mask codes need a kernel volume <= 32, got %d", V);
    FGX_CHECK_ARG(n < 0xFFFFFFFFull, "fgx_subm_neighbor_map_sorted: row indices must fit below 2^32-1");
    if (n == 0) return FGX_OK;
    const long double vol_ld = (long double)B * W * H * D;
    FGX_CHECK_ARG(vol_ld <= (key_bits == 32 ? 4294967296.0L : 9223372036854775808.0L),
                  "fgx_subm_neighbor_map_sorted: the grid needs wider keys than %d bits", key_bits);
    const uint64_t vol = (uint64_t)B * (uint64_t)W * (uint64_t)H * (uint64_t)D;
    SortedLayout L = sorted_layout(n, key_bits, Kw * Kh);
    FGX_CHECK_ARG(coords && out_map && workspace, "fgx_subm_neighbor_map_sorted: null buffer");
    FGX_CHECK_ARG(((uintptr_t)coords & 15) == 0, "fgx_subm_neighbor_map_sorted: coords must be 16-byte aligned");
    FGX_CHECK_ARG(workspace_bytes >= L.total, "fgx_subm_neighbor_map_sorted: workspace of %zu bytes, need %zu", workspace_bytes, L.total);
    FGX_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fgx_subm_neighbor_map_sorted: workspace must be 256-byte aligned");
    SubmGeom g{W, H, D, Kw, Kh, Kd, V, Dw, Dh, Dd};
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)workspace;
    return key_bits == 32 ? build_sorted<uint32_t>(coords, n, vol, g, ws, L, out_map, gray, binary, s)
                          : build_sorted<uint64_t>(coords, n, vol, g, ws, L, out_map, gray, binary, s);
}

}  // extern "C"
