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
#include "radix_sort.h"

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

// flat_keys_kernel that also tells whether the keys ascend as the voxels come: descents[0] = 1 when some voxel's key is
// smaller than its predecessor's (the word is cleared by a kernel before this one)
template <typename K>
__global__ void __launch_bounds__(256) flat_keys_check_kernel(const int32_t* __restrict__ coords, size_t n, int W, int H, int D,
                                                              K* __restrict__ keys, uint32_t* __restrict__ rows,
                                                              uint32_t* __restrict__ descents) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int4 c = reinterpret_cast<const int4*>(coords)[i];
    const uint64_t kc = (((uint64_t)(uint32_t)c.x * (uint64_t)W + (uint64_t)c.y) * (uint64_t)H + (uint64_t)c.z) * (uint64_t)D + (uint64_t)c.w;
    keys[i] = (K)kc;
    rows[i] = (uint32_t)i;
    if (i > 0) {
        const int4 a = reinterpret_cast<const int4*>(coords)[i - 1];
        const uint64_t ka = (((uint64_t)(uint32_t)a.x * (uint64_t)W + (uint64_t)a.y) * (uint64_t)H + (uint64_t)a.z) * (uint64_t)D + (uint64_t)a.w;
        if (kc < ka) descents[0] = 1u;      // (every writer stores the same value)
    }
}

// descents[0] = 1 when some voxel's flattened key is smaller than its predecessor's (the caller clears the word first)
__global__ void __launch_bounds__(256) key_order_kernel(const int32_t* __restrict__ coords, size_t n, int W, int H, int D,
                                                        uint32_t* __restrict__ descents) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i == 0 || i >= n) return;
    const int4 a = reinterpret_cast<const int4*>(coords)[i - 1], c = reinterpret_cast<const int4*>(coords)[i];
    const uint64_t ka = (((uint64_t)(uint32_t)a.x * (uint64_t)W + (uint64_t)a.y) * (uint64_t)H + (uint64_t)a.z) * (uint64_t)D + (uint64_t)a.w;
    const uint64_t kc = (((uint64_t)(uint32_t)c.x * (uint64_t)W + (uint64_t)c.y) * (uint64_t)H + (uint64_t)c.z) * (uint64_t)D + (uint64_t)c.w;
    if (kc < ka) descents[0] = 1u;      // (every writer stores the same value)
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
// (`pick` != nullptr: the sorted keys are `skeys` when that word is non-zero and `skeys_if_not` when it is zero -- the
// key sort ahead of this kernel was conditional on the same word)
template <typename K>
__global__ void __launch_bounds__(256) window_bounds_kernel(const K* __restrict__ skeys, size_t n, unsigned long long vol,
                                                            SubmGeom g, unsigned groups, uint32_t* __restrict__ bounds,
                                                            const uint32_t* __restrict__ pick, const K* __restrict__ skeys_if_not) {
    if (pick != nullptr && *pick == 0u) skeys = skeys_if_not;
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

// Which rows hold the keys first, first + Dd, ... (Kd of them, ascending) in the sorted window wkeys[0, wn), wn > 0?
// emit(kz, row index or EMPTY) is called for every kz.  One binary search for the first key -- a fixed number of
// halving steps, the same for every lane, no data-dependent branch -- then at most Dd steps forward to each next one
// (keys are distinct integers).  `first` may lie below zero (next to the origin, or for a base cell outside the grid);
// row_in tells whether the (x, y) of these targets lies inside the grid, target kz lies inside along z when
// z_first + kz * Dd is in [0, D).  A lane outside searches too and discards what it finds.
template <typename K, typename Emit>
__device__ __forceinline__ void search_staged(const K* wkeys, const uint32_t* wrows, unsigned wn, long long first, bool row_in,
                                              int z_first, int Kd, int Dd, int D, Emit emit) {
    const K t0 = (K)(first < 0 ? 0 : first);
    unsigned pos = 0;           // number of window keys below the current target
    for (unsigned step = 1u << (31 - __clz((int)wn)); step > 0; step >>= 1) {
        const unsigned cand = pos + step;
        const unsigned at = (cand <= wn ? cand : wn) - 1;
        if (wkeys[at] < t0 && cand <= wn) pos = cand;
    }
    for (int kz = 0; kz < Kd; ++kz) {
        const long long t = first + (long long)kz * Dd;
        const K tk = (K)t;
        if (kz > 0 && t > 0) {
            for (int s = 0; s < Dd; ++s) {
                const unsigned at = pos < wn ? pos : wn - 1;
                if (wkeys[at] < tk && pos < wn) ++pos;
            }
            // Only a window with repeated keys (the same voxel given twice) can still be short of the target:
            // finish with a search over the rest.
            if (pos < wn && wkeys[pos] < tk) {
                unsigned lo = pos + 1, hi = wn;
                while (lo < hi) {
                    const unsigned mid = (lo + hi) >> 1;
                    if (wkeys[mid] < tk) lo = mid + 1;
                    else hi = mid;
                }
                pos = lo;
            }
        }
        const unsigned at = pos < wn ? pos : wn - 1;
        const int z2 = z_first + kz * Dd;
        const bool hit = wkeys[at] == tk && pos < wn && t >= 0 && row_in && z2 >= 0 && z2 < D;
        emit(kz, hit ? wrows[at] : FGX_EMPTY32);
    }
}

// The same questions for a window that is too long for LDS (or empty): searched where it lies in memory.
template <typename K, typename Emit>
__device__ __forceinline__ void search_in_place(const K* __restrict__ skeys, const uint32_t* __restrict__ srows, size_t lo,
                                                size_t hi, long long first, bool row_in, int z_first, int Kd, int Dd, int D,
                                                Emit emit) {
    for (int kz = 0; kz < Kd; ++kz) {
        const long long t = first + (long long)kz * Dd;
        const int z2 = z_first + kz * Dd;
        uint32_t value = FGX_EMPTY32;
        if (lo < hi && row_in && z2 >= 0 && z2 < D && t >= 0) {
            const size_t q = lower_bound_at<K>(skeys, lo, hi, (K)t);
            if (q < hi && skeys[q] == (K)t) value = srows[q];
        }
        emit(kz, value);
    }
}

template <typename K>
__global__ void __launch_bounds__(kGroup) merge_neighbor_kernel(const K* __restrict__ skeys, const uint32_t* __restrict__ srows,
                                                                const uint32_t* __restrict__ bounds, size_t n, SubmGeom g,
                                                                uint32_t* __restrict__ out_map,
                                                                int32_t* __restrict__ gray, int32_t* __restrict__ binary,
                                                                const uint32_t* __restrict__ pick, const K* __restrict__ skeys_if_not,
                                                                const uint32_t* __restrict__ srows_if_not) {
    if (pick != nullptr && *pick == 0u) {       // (as in window_bounds_kernel)
        skeys = skeys_if_not;
        srows = srows_if_not;
    }
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
        if constexpr (sizeof(K) == 4) {         // 32-bit division is several times shorter than the 64-bit sequence
            uint32_t t = (uint32_t)key;
            z = (int)(t % (uint32_t)g.D);
            t /= (uint32_t)g.D;
            y = (int)(t % (uint32_t)g.H);
            t /= (uint32_t)g.H;
            x = (int)(t % (uint32_t)g.W);
        } else {
            uint64_t t = (uint64_t)key;
            z = (int)(t % (uint64_t)g.D);
            t /= (uint64_t)g.D;
            y = (int)(t % (uint64_t)g.H);
            t /= (uint64_t)g.H;
            x = (int)(t % (uint64_t)g.W);
        }
    }
    __syncthreads();

    // The windows of the next kAhead (dx, dy) rows travel from memory to registers together, so their latencies overlap;
    // each is then put into LDS and searched in turn.
    constexpr int kAhead = 9;
    K pk[kAhead][kPer];
    uint32_t pr[kAhead][kPer];
    uint32_t mask = 0;
    const int z_first = z - (g.Kd / 2) * g.Dd;
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
                const long long first = (long long)key + off - (long long)(g.Kd / 2) * g.Dd;
                auto emit = [&](int kz, uint32_t value) {
                    const int v = r * g.Kd + kz;
                    if (v == g.V / 2) value = me;       // the middle entry is the voxel itself, found or not (subm_neighbor_map.cu:64-66)
                    out_row[kz] = value;
                    if (v < 32 && value != FGX_EMPTY32) mask |= 1u << v;
                };
                if (staged && w > 0) search_staged<K>(wkeys, wrows, (unsigned)w, first, row_in, z_first, g.Kd, g.Dd, g.D, emit);
                else search_in_place<K>(skeys, srows, lo, hi, first, row_in, z_first, g.Kd, g.Dd, g.D, emit);
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

__global__ void __launch_bounds__(256) fill_words_kernel(uint32_t* p, size_t count, uint32_t value) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    for (; i < count; i += stride) p[i] = value;
}

struct SortedLayout {
    size_t keys_in, keys_out, rows_in, rows_out, bounds, temp, temp_bytes, radix, flag, total;
};

// up to this many voxels with 32-bit keys the key sort can be left to the device (radix_sort.h with its run_if word)
constexpr size_t kDeviceDecidesMax = 2097152;

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
    off += align_up(L.temp_bytes, 256);
    L.flag = off;
    off += 256;
    L.radix = off;
    if (key_bits == 32 && n <= kDeviceDecidesMax) off += radix_layout(n).total;
    L.total = off;
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

// presorted: 0 = sort the keys, 1 = the caller knows that they ascend as the voxels come, 2 = find out on the device
template <typename K>
int build_sorted(const int32_t* coords, size_t n, uint64_t vol, const SubmGeom& g, int presorted, char* ws, const SortedLayout& L,
                 uint32_t* out_map, int32_t* gray, int32_t* binary, hipStream_t s) {
    K* keys_in = (K*)(ws + L.keys_in);
    K* keys_out = (K*)(ws + L.keys_out);
    uint32_t* rows_in = (uint32_t*)(ws + L.rows_in);
    uint32_t* rows_out = (uint32_t*)(ws + L.rows_out);
    const K* skeys = keys_out;
    const uint32_t* srows = rows_out;
    const uint32_t* pick = nullptr;         // device word: 0 = the voxels came in key order and nothing was sorted
    PhaseEnd phases{s};
    unsigned end_bit = bit_length(vol - 1);
    if (end_bit == 0) end_bit = 1;
    if (presorted == 1) {   // keys ascend as the voxels come: the sorted arrays are the keys and 0, 1, 2, ... themselves
        phase_mark("keys", s);
        flat_keys_kernel<K><<<cdiv(n, 256), 256, 0, s>>>(coords, n, g.W, g.H, g.D, keys_out, rows_out);
        FGX_CHECK_LAUNCH("fgx_subm_neighbor_map_sorted(keys)");
    } else if (presorted == 2 && sizeof(K) == 4 && n <= kDeviceDecidesMax) {
        // Voxels that already come in scan order (a dense grid's nonzero(), a sorted voxelizer) need no key sort.  Whether
        // they do is found while the keys are made; the sort's kernels return at once when they do, and the kernels after
        // it take the unsorted arrays then -- no answer has to travel to the host.
        uint32_t* flag = (uint32_t*)(ws + L.flag);
        phase_mark("keys", s);
        fill_words_kernel<<<1, 64, 0, s>>>(flag, 1, 0u);
        FGX_CHECK_LAUNCH("fgx_subm_neighbor_map_sorted(flag)");
        flat_keys_check_kernel<K><<<cdiv(n, 256), 256, 0, s>>>(coords, n, g.W, g.H, g.D, keys_in, rows_in, flag);
        FGX_CHECK_LAUNCH("fgx_subm_neighbor_map_sorted(keys)");
        phase_mark("key sort", s);
        const uint32_t *ks = nullptr, *vs = nullptr;
        int rc = radix_sort_pairs_u32((const uint32_t*)keys_in, nullptr, n, end_bit, ws + L.radix, radix_layout(n), &ks, &vs, nullptr,
                                      s, "fgx_subm_neighbor_map_sorted(key sort)", flag);
        if (rc != FGX_OK) return rc;
        skeys = (const K*)ks;
        srows = vs;
        pick = flag;
    } else {
        phase_mark("key sort", s);
        flat_keys_kernel<K><<<cdiv(n, 256), 256, 0, s>>>(coords, n, g.W, g.H, g.D, keys_in, rows_in);
        FGX_CHECK_LAUNCH("fgx_subm_neighbor_map_sorted(keys)");
        size_t temp_bytes = L.temp_bytes;
        FGX_CHECK_HIP(rocprim::radix_sort_pairs(ws + L.temp, temp_bytes, (const K*)keys_in, keys_out, (const uint32_t*)rows_in, rows_out,
                                                n, 0u, end_bit, s));
    }
    const unsigned groups = cdiv(n, kGroup);
    uint32_t* bounds = (uint32_t*)(ws + L.bounds);
    phase_mark("window bounds", s);
    window_bounds_kernel<K><<<cdiv((size_t)groups * g.Kw * g.Kh * 2, 256), 256, 0, s>>>(skeys, n, (unsigned long long)vol, g, groups, bounds,
                                                                                        pick, (const K*)keys_in);
    FGX_CHECK_LAUNCH("fgx_subm_neighbor_map_sorted(bounds)");
    phase_mark("merge", s);
    merge_neighbor_kernel<K><<<groups, kGroup, 0, s>>>(skeys, srows, bounds, n, g, out_map, gray, binary, pick, (const K*)keys_in,
                                                       (const uint32_t*)rows_in);
    FGX_CHECK_LAUNCH("fgx_subm_neighbor_map_sorted");
    return FGX_OK;
}

// ------------------------------------------------------------------------------------------------
// Generic sparse convolution: the same search with the OUTPUT voxels as queries.
//
// Output voxel o = (b, x, y, z) reads the input voxel at (x*Sw - Pw + kx*Dw, ...): for a fixed kernel position that is its
// "base" cell (x*Sw - Pw, y*Sh - Ph, z*Sd - Pd) plus a constant, and in flattened input keys base(o) + constant, even when
// the base cell itself lies outside the grid (the sum is linear).  So the queries are sorted by base(o) (biased to be
// non-negative), and a group of 256 consecutive ones again finds all its (kx, ky) neighbors in one window of the sorted
// input keys.  A query that cannot reach the grid at all (any base coordinate further out than the kernel spans, or a
// batch index outside [0, B)) gets the largest key and an all-empty row.
// ------------------------------------------------------------------------------------------------
struct ConvGeomS {
    int B, W, H, D;
    int Kw, Kh, Kd, V;
    int Sw, Sh, Sd;
    int Pw, Ph, Pd;
    int Dw, Dh, Dd;
};

__device__ __forceinline__ bool query_base(const int4 c, const ConvGeomS& g, int& xi, int& yi, int& zi, long long& base) {
    xi = c.y * g.Sw - g.Pw;
    yi = c.z * g.Sh - g.Ph;
    zi = c.w * g.Sd - g.Pd;
    base = (((long long)c.x * g.W + xi) * g.H + yi) * g.D + zi;
    return c.x >= 0 && c.x < g.B && xi > -g.Kw * g.Dw && xi < g.W && yi > -g.Kh * g.Dh && yi < g.H && zi > -g.Kd * g.Dd && zi < g.D;
}

__global__ void __launch_bounds__(256) query_keys_kernel(const int32_t* __restrict__ out_coords, size_t n_out, ConvGeomS g,
                                                         unsigned long long bias, unsigned long long dead_key,
                                                         uint64_t* __restrict__ keys, uint32_t* __restrict__ rows) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n_out) return;
    int xi, yi, zi;
    long long base;
    const bool live = query_base(reinterpret_cast<const int4*>(out_coords)[i], g, xi, yi, zi, base);
    keys[i] = live ? (uint64_t)(base + (long long)bias) : (uint64_t)dead_key;
    rows[i] = (uint32_t)i;
}

// as window_bounds_kernel, with the group's range taken from the sorted query keys (dead queries, at the end, excluded)
template <typename K>
__global__ void __launch_bounds__(256) query_bounds_kernel(const K* __restrict__ skeys, size_t n_in, unsigned long long vol,
                                                           const uint64_t* __restrict__ qkeys, size_t n_out,
                                                           unsigned long long bias, unsigned long long dead_key, ConvGeomS g,
                                                           unsigned groups, uint32_t* __restrict__ bounds) {
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int R = g.Kw * g.Kh;
    if (t >= (size_t)groups * R * 2) return;
    const size_t grp = t / (2 * R);
    const int r = (int)(t % (2 * R)) >> 1;
    const size_t p0 = grp * kGroup;
    size_t p1 = (n_out - p0 < (size_t)kGroup ? n_out : p0 + kGroup) - 1;      // last query of the group
    uint32_t pos = 0;
    if (qkeys[p0] != dead_key) {
        // the last live query of the group (dead keys are the largest)
        if (qkeys[p1] == dead_key) p1 = lower_bound_at<uint64_t>(qkeys, p0, p1, dead_key) - 1;
        const long long HD = (long long)g.H * g.D;
        const long long off = (long long)(r / g.Kh) * g.Dw * HD + (long long)(r % g.Kh) * g.Dh * g.D;
        const long long lo_t = (long long)(qkeys[p0] - bias) + off, hi_t = (long long)(qkeys[p1] - bias) + off + (long long)(g.Kd - 1) * g.Dd;
        if ((t & 1) == 0) pos = (uint32_t)(hi_t < 0 ? 0 : (lo_t >= (long long)vol ? n_in : lower_bound_at<K>(skeys, 0, n_in, (K)(lo_t < 0 ? 0 : lo_t))));
        else pos = (uint32_t)(hi_t < 0 ? 0 : (hi_t + 1 >= (long long)vol ? n_in : lower_bound_at<K>(skeys, 0, n_in, (K)(hi_t + 1))));
    }
    bounds[t] = pos;
}

template <typename K>
__global__ void __launch_bounds__(kGroup) merge_query_kernel(const K* __restrict__ skeys, const uint32_t* __restrict__ srows,
                                                             const uint64_t* __restrict__ qkeys, const uint32_t* __restrict__ qrows,
                                                             const int32_t* __restrict__ out_coords, const uint32_t* __restrict__ bounds,
                                                             size_t n_out, unsigned long long dead_key, ConvGeomS g,
                                                             uint32_t* __restrict__ map_fwd, uint32_t* __restrict__ map_bwd,
                                                             int32_t* __restrict__ gray, int32_t* __restrict__ binary) {
    constexpr int kPer = kWindow / kGroup;
    __shared__ K wkeys[kWindow];
    __shared__ uint32_t wrows[kWindow];
    __shared__ uint32_t win_lo[kMaxRows], win_hi[kMaxRows];
    __shared__ uint32_t out_rows[kGroup * (kStageV + 1)];
    __shared__ uint32_t out_dst[kGroup];
    const bool stage_out = g.V <= kStageV;
    const size_t p0 = (size_t)blockIdx.x * kGroup;
    const int cnt = (int)(n_out - p0 < (size_t)kGroup ? n_out - p0 : (size_t)kGroup);
    const int tid = threadIdx.x;
    const bool present = tid < cnt;
    const int R = g.Kw * g.Kh;
    const long long HD = (long long)g.H * g.D;
    for (int j = tid; j < R; j += kGroup) {
        win_lo[j] = bounds[((size_t)blockIdx.x * R + j) * 2];
        win_hi[j] = bounds[((size_t)blockIdx.x * R + j) * 2 + 1];
    }
    uint32_t me = 0;
    int xi = 0, yi = 0, zi = 0;
    long long base = 0;
    bool live = false;
    if (present) {
        me = qrows[p0 + tid];
        live = qkeys[p0 + tid] != dead_key;
        bool ok = query_base(reinterpret_cast<const int4*>(out_coords)[me], g, xi, yi, zi, base);
        live = live && ok;
    }
    __syncthreads();

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
            if (w > (size_t)kWindow) continue;
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
            if (present) {
                const int kx = r / g.Kh, ky = r % g.Kh;
                const int x2 = xi + kx * g.Dw, y2 = yi + ky * g.Dh;
                const bool row_in = live && x2 >= 0 && x2 < g.W && y2 >= 0 && y2 < g.H;
                const long long off = (long long)kx * g.Dw * HD + (long long)ky * g.Dh * g.D;
                uint32_t* out_row = stage_out ? out_rows + tid * (kStageV + 1) + r * g.Kd
                                              : map_fwd + (size_t)me * g.V + (size_t)r * g.Kd;
                auto emit = [&](int kz, uint32_t value) {
                    out_row[kz] = value;
                    const int v = r * g.Kd + kz;
                    if (value != FGX_EMPTY32) {
                        if (v < 32) mask |= 1u << v;
                        if (map_bwd != nullptr) map_bwd[(size_t)value * g.V + v] = me;
                    }
                };
                if (staged && w > 0) search_staged<K>(wkeys, wrows, (unsigned)w, base + off, row_in, zi, g.Kd, g.Dd, g.D, emit);
                else search_in_place<K>(skeys, srows, lo, hi, base + off, row_in, zi, g.Kd, g.Dd, g.D, emit);
            }
            __syncthreads();
        }
    }
    if (present && gray != nullptr) {
        gray[me] = (int32_t)mask;
        binary[me] = (int32_t)gray_decode(mask);
    }
    if (stage_out) {
        out_dst[tid] = me;
        __syncthreads();
        const int lane32 = tid & 31;
        for (int row = tid >> 5; row < cnt; row += kGroup / 32)
            if (lane32 < g.V) map_fwd[(size_t)out_dst[row] * g.V + lane32] = out_rows[row * (kStageV + 1) + lane32];
    }
}


struct QueryLayout {
    SortedLayout in;            // the input voxels' sort (bounds sized for the query groups)
    size_t qkeys_in, qkeys_out, qrows_in, qrows_out, qtemp, qtemp_bytes, total;
};

QueryLayout query_layout(size_t n_in, size_t n_out, int key_bits, int rows_xy) {
    QueryLayout Q{};
    Q.in = sorted_layout(n_in, key_bits, 0);
    size_t off = Q.in.total;
    const size_t nq = n_out ? n_out : 1;
    Q.qkeys_in = off;
    off = align_up(off + nq * 8, 256);
    Q.qkeys_out = off;
    off = align_up(off + nq * 8, 256);
    Q.qrows_in = off;
    off = align_up(off + nq * 4, 256);
    Q.qrows_out = off;
    off = align_up(off + nq * 4, 256);
    Q.in.bounds = off;
    off = align_up(off + (size_t)cdiv(nq, kGroup) * rows_xy * 2 * sizeof(uint32_t), 256);
    Q.qtemp = off;
    Q.qtemp_bytes = pair_sort_temp_bytes<uint64_t>(n_out);
    Q.total = off + align_up(Q.qtemp_bytes, 256);
    return Q;
}

template <typename K>
int build_query_sorted(const int32_t* in_coords, size_t n_in, const int32_t* out_coords, size_t n_out, uint64_t vol,
                       const ConvGeomS& g, char* ws, const QueryLayout& Q, uint32_t* map_fwd, uint32_t* map_bwd, int32_t* gray,
                       int32_t* binary, hipStream_t s) {
    K* keys_in = (K*)(ws + Q.in.keys_in);
    K* keys_out = (K*)(ws + Q.in.keys_out);
    uint32_t* rows_in = (uint32_t*)(ws + Q.in.rows_in);
    uint32_t* rows_out = (uint32_t*)(ws + Q.in.rows_out);
    flat_keys_kernel<K><<<cdiv(n_in, 256), 256, 0, s>>>(in_coords, n_in, g.W, g.H, g.D, keys_in, rows_in);
    FGX_CHECK_LAUNCH("fgx_spconv_neighbor_map_sorted(keys)");
    size_t temp_bytes = Q.in.temp_bytes;
    unsigned end_bit = bit_length(vol - 1);
    if (end_bit == 0) end_bit = 1;
    FGX_CHECK_HIP(rocprim::radix_sort_pairs(ws + Q.in.temp, temp_bytes, (const K*)keys_in, keys_out, (const uint32_t*)rows_in, rows_out,
                                            n_in, 0u, end_bit, s));
    // queries: base keys biased by the furthest a live base cell can lie below the grid origin
    const long long HD = (long long)g.H * g.D;
    const unsigned long long bias = (unsigned long long)((long long)g.Kw * g.Dw * HD + (long long)g.Kh * g.Dh * g.D + (long long)g.Kd * g.Dd);
    const unsigned long long dead_key = vol + 2 * bias + 1;
    uint64_t* qkeys_in = (uint64_t*)(ws + Q.qkeys_in);
    uint64_t* qkeys_out = (uint64_t*)(ws + Q.qkeys_out);
    uint32_t* qrows_in = (uint32_t*)(ws + Q.qrows_in);
    uint32_t* qrows_out = (uint32_t*)(ws + Q.qrows_out);
    query_keys_kernel<<<cdiv(n_out, 256), 256, 0, s>>>(out_coords, n_out, g, bias, dead_key, qkeys_in, qrows_in);
    FGX_CHECK_LAUNCH("fgx_spconv_neighbor_map_sorted(query keys)");
    temp_bytes = Q.qtemp_bytes;
    FGX_CHECK_HIP(rocprim::radix_sort_pairs(ws + Q.qtemp, temp_bytes, (const uint64_t*)qkeys_in, qkeys_out, (const uint32_t*)qrows_in,
                                            qrows_out, n_out, 0u, bit_length(dead_key), s));
    const unsigned groups = cdiv(n_out, kGroup);
    uint32_t* bounds = (uint32_t*)(ws + Q.in.bounds);
    query_bounds_kernel<K><<<cdiv((size_t)groups * g.Kw * g.Kh * 2, 256), 256, 0, s>>>(keys_out, n_in, (unsigned long long)vol, qkeys_out,
                                                                                      n_out, bias, dead_key, g, groups, bounds);
    FGX_CHECK_LAUNCH("fgx_spconv_neighbor_map_sorted(bounds)");
    merge_query_kernel<K><<<groups, kGroup, 0, s>>>(keys_out, rows_out, qkeys_out, qrows_out, out_coords, bounds, n_out, dead_key, g,
                                                    map_fwd, map_bwd, gray, binary);
    FGX_CHECK_LAUNCH("fgx_spconv_neighbor_map_sorted");
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

int fgx_coords_key_order(const int32_t* coords, size_t n, int W, int H, int D, uint32_t* descents, fgx_stream_t stream) {
    FGX_CHECK_ARG(W > 0 && H > 0 && D > 0, "fgx_coords_key_order: grid extents must be positive");
    FGX_CHECK_ARG(descents != nullptr && (n == 0 || coords != nullptr), "fgx_coords_key_order: null buffer");
    FGX_CHECK_ARG(((uintptr_t)coords & 15) == 0, "fgx_coords_key_order: coords must be 16-byte aligned");
    if (n < 2) return FGX_OK;
    hipStream_t s = (hipStream_t)stream;
    PhaseEnd phases{s};
    phase_mark("key order check", s);
    key_order_kernel<<<cdiv(n, 256), 256, 0, s>>>(coords, n, W, H, D, descents);
    FGX_CHECK_LAUNCH("fgx_coords_key_order");
    return FGX_OK;
}

int fgx_subm_neighbor_map_sorted(const int32_t* coords, size_t n, int B, int W, int H, int D, int Kw, int Kh, int Kd, int Dw,
                                 int Dh, int Dd, int key_bits, int presorted, void* workspace, size_t workspace_bytes,
                                 uint32_t* out_map, int32_t* gray, int32_t* binary, fgx_stream_t stream) {
    FGX_CHECK_ARG(key_bits == 32 || key_bits == 64, "fgx_subm_neighbor_map_sorted: key_bits must be 32 or 64, got %d", key_bits);
    FGX_CHECK_ARG(presorted >= 0 && presorted <= 2, "fgx_subm_neighbor_map_sorted: presorted must be 0, 1 or 2, got %d", presorted);
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
    return key_bits == 32 ? build_sorted<uint32_t>(coords, n, vol, g, presorted, ws, L, out_map, gray, binary, s)
                          : build_sorted<uint64_t>(coords, n, vol, g, presorted, ws, L, out_map, gray, binary, s);
}

size_t fgx_spconv_neighbor_map_sorted_workspace_bytes(size_t n_in, size_t n_out, int key_bits, int Kw, int Kh) {
    if ((key_bits != 32 && key_bits != 64) || Kw < 1 || Kh < 1 || Kw * Kh > kMaxRows) return 0;
    return query_layout(n_in, n_out, key_bits, Kw * Kh).total;
}

int fgx_spconv_neighbor_map_sorted(const int32_t* in_coords, size_t n_in, const int32_t* out_coords, size_t n_out, int B, int W,
                                   int H, int D, int Kw, int Kh, int Kd, int Sw, int Sh, int Sd, int Pw, int Ph, int Pd, int Dw,
                                   int Dh, int Dd, int key_bits, void* workspace, size_t workspace_bytes, uint32_t* map_fwd,
                                   uint32_t* map_bwd, int32_t* gray, int32_t* binary, fgx_stream_t stream) {
    FGX_CHECK_ARG(key_bits == 32 || key_bits == 64, "fgx_spconv_neighbor_map_sorted: key_bits must be 32 or 64, got %d", key_bits);
    FGX_CHECK_ARG(B > 0 && W > 0 && H > 0 && D > 0, "fgx_spconv_neighbor_map_sorted: grid extents must be positive");
    FGX_CHECK_ARG(Kw > 0 && Kh > 0 && Kd > 0 && Sw > 0 && Sh > 0 && Sd > 0 && Dw > 0 && Dh > 0 && Dd > 0 && Pw >= 0 && Ph >= 0 && Pd >= 0,
                  "fgx_spconv_neighbor_map_sorted: bad kernel geometry");
    FGX_CHECK_ARG(Kw * Kh <= kMaxRows && (long long)Kw * Kh * Kd <= 1 << 20, "fgx_spconv_neighbor_map_sorted: kernel too large");
    const int V = Kw * Kh * Kd;
    FGX_CHECK_ARG((gray == nullptr) == (binary == nullptr), "fgx_spconv_neighbor_map_sorted: gray and binary go together");
    FGX_CHECK_ARG(gray == nullptr || V <= 32, "fgx_spconv_neighbor_map_sorted: mask codes need a kernel volume <= 32, got %d", V);
    FGX_CHECK_ARG(n_in < 0xFFFFFFFFull && n_out < 0xFFFFFFFFull, "fgx_spconv_neighbor_map_sorted: row indices must fit below 2^32-1");
    const long double vol_ld = (long double)B * W * H * D;
    FGX_CHECK_ARG(vol_ld <= (key_bits == 32 ? 4294967296.0L : 4611686018427387904.0L),
                  "fgx_spconv_neighbor_map_sorted: the grid needs wider keys than %d bits", key_bits);
    hipStream_t s = (hipStream_t)stream;
    if (map_bwd != nullptr && n_in > 0) {
        const size_t cells = n_in * (size_t)V;
        unsigned grid = cdiv(cells, 256);
        if (grid > 65536u) grid = 65536u;
        fill_words_kernel<<<grid, 256, 0, s>>>(map_bwd, cells, FGX_EMPTY32);
        FGX_CHECK_LAUNCH("fgx_spconv_neighbor_map_sorted(fill)");
    }
    if (n_out == 0) return FGX_OK;
    FGX_CHECK_ARG(out_coords && map_fwd, "fgx_spconv_neighbor_map_sorted: null buffer");
    FGX_CHECK_ARG(((uintptr_t)out_coords & 15) == 0 && ((uintptr_t)in_coords & 15) == 0, "fgx_spconv_neighbor_map_sorted: coords must be 16-byte aligned");
    if (n_in == 0) {
        const size_t cells = n_out * (size_t)V;
        unsigned grid = cdiv(cells, 256);
        if (grid > 65536u) grid = 65536u;
        fill_words_kernel<<<grid, 256, 0, s>>>(map_fwd, cells, FGX_EMPTY32);
        if (gray != nullptr) {
            fill_words_kernel<<<cdiv(n_out, 256), 256, 0, s>>>((uint32_t*)gray, n_out, 0u);
            fill_words_kernel<<<cdiv(n_out, 256), 256, 0, s>>>((uint32_t*)binary, n_out, 0u);
        }
        FGX_CHECK_LAUNCH("fgx_spconv_neighbor_map_sorted(fill)");
        return FGX_OK;
    }
    FGX_CHECK_ARG(in_coords && workspace, "fgx_spconv_neighbor_map_sorted: null buffer");
    QueryLayout Q = query_layout(n_in, n_out, key_bits, Kw * Kh);
    FGX_CHECK_ARG(workspace_bytes >= Q.total, "fgx_spconv_neighbor_map_sorted: workspace of %zu bytes, need %zu", workspace_bytes, Q.total);
    FGX_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fgx_spconv_neighbor_map_sorted: workspace must be 256-byte aligned");
    const uint64_t vol = (uint64_t)B * (uint64_t)W * (uint64_t)H * (uint64_t)D;
    ConvGeomS g{B, W, H, D, Kw, Kh, Kd, V, Sw, Sh, Sd, Pw, Ph, Pd, Dw, Dh, Dd};
    char* ws = (char*)workspace;
    return key_bits == 32 ? build_query_sorted<uint32_t>(in_coords, n_in, out_coords, n_out, vol, g, ws, Q, map_fwd, map_bwd, gray, binary, s)
                          : build_query_sorted<uint64_t>(in_coords, n_in, out_coords, n_out, vol, g, ws, Q, map_fwd, map_bwd, gray, binary, s);
}

}  // extern "C"
