// Post-processing of the neighbor map for the masked implicit GEMM on gfx950:
// mask-sorted voxel order, (v, n)-ordered pair lists for wgrad, per-tile offset masks.
//
// Departures from the reference's data flow (flex_gemm/kernels/cuda/spconv/migemm_neighmap_pp.cu):
//   * pair lists are built from the 4-byte validity masks with a per-block count, one device scan
//     over [V, blocks] and a rank-and-write pass, instead of materialising a transposed map, a
//     transposed 0/1 mask and their N*V-long prefix sum (:85-154, :224-225);
//   * the sort is a stable LSD radix sort restricted to the V mask bits;
//   * tile masks are OR-reduced one wavefront per tile with cross-lane shuffles and accept any
//     tile size, not only powers of two.
#include <cstring>
#include <string.h>

#include <rocprim/rocprim.hpp>

#include "fgx_common.h"
#include "radix_sort.h"

namespace fgx {
namespace {

constexpr int kBlock = 256;
constexpr int kPairRows = 256;       // voxels per block in the pair-list passes (larger blocks were not faster)
constexpr int kPairThreads = 256;    // ... walked in chunks of this many

__global__ void __launch_bounds__(kBlock) iota_u32_kernel(uint32_t* out, size_t n) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) out[i] = (uint32_t)i;
}

__global__ void __launch_bounds__(kBlock) widen_u32_i64_kernel(const uint32_t* in, int64_t* out, size_t n) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) out[i] = (int64_t)in[i];
}

// 16 bits of x, y, z interleaved (x highest), batch index on top: voxels close in space get close keys
__device__ __forceinline__ uint64_t spread16(uint32_t x) {
    uint64_t v = x & 0xFFFFu;
    v = (v | (v << 16)) & 0x0000FF0000FFull;
    v = (v | (v << 8)) & 0x00F00F00F00Full;
    v = (v | (v << 4)) & 0x0C30C30C30C3ull;
    v = (v | (v << 2)) & 0x249249249249ull;
    return v;
}

// Z-order key: the batch index right above the 3 * bits interleaved coordinate bits (Key: 32 bits when they all fit)
template <typename Key>
__global__ void __launch_bounds__(kBlock) morton_key_packed_kernel(const int32_t* __restrict__ coords, size_t n, int bits,
                                                                   Key* __restrict__ keys, uint32_t* __restrict__ vals) {
    size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    int4 c = reinterpret_cast<const int4*>(coords)[i];
    const uint64_t m = (spread16((uint32_t)c.y) << 2) | (spread16((uint32_t)c.z) << 1) | spread16((uint32_t)c.w);
    keys[i] = (Key)(((uint64_t)(uint32_t)c.x << (3 * bits)) | (m & ((1ull << (3 * bits)) - 1ull)));
    vals[i] = (uint32_t)i;
}

// position p of the spatial order -> (chunk of p, mask code of its voxel)
__global__ void __launch_bounds__(kBlock) chunk_code_key_kernel(const uint32_t* __restrict__ perm,
                                                                const int32_t* __restrict__ binary, size_t n,
                                                                uint32_t chunk_rows, int code_bits, uint64_t* __restrict__ keys) {
    size_t p = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (p >= n) return;
    keys[p] = ((uint64_t)(p / chunk_rows) << code_bits) | (uint32_t)binary[perm[p]];
}

struct LocalityLayout {
    size_t keys_a, keys_b, vals_a, vals_b, temp, temp_bytes, total;
};

LocalityLayout locality_layout(size_t n) {
    LocalityLayout L{};
    size_t nn = n ? n : 1;
    size_t temp_bytes = 0;
    (void)rocprim::radix_sort_pairs(nullptr, temp_bytes, (const uint64_t*)nullptr, (uint64_t*)nullptr,
                                    (const uint32_t*)nullptr, (uint32_t*)nullptr, nn, 0u, 64u, (hipStream_t)0);
    size_t off = 0;
    L.keys_a = off; off = align_up(off + nn * 8, 256);
    L.keys_b = off; off = align_up(off + nn * 8, 256);
    L.vals_a = off; off = align_up(off + nn * 4, 256);
    L.vals_b = off; off = align_up(off + nn * 4, 256);
    L.temp = off;   off = align_up(off + temp_bytes, 256);
    L.temp_bytes = temp_bytes;
    L.total = off;
    return L;
}

int bits_for(size_t x) {   // smallest b with 2^b > x
    int b = 0;
    while (b < 63 && ((size_t)1 << b) <= x) ++b;
    return b;
}


// The mask sort: between these sizes the radix sort of radix_sort.h is ahead of the library's (measured, 27-bit keys:
// 0.095 against 0.154 ms at 669 288 items; 0.077 against 0.068 ms at 166 232, where the library sorts blocks and merges
// them; 0.189 against 0.182 ms at 2 667 120, where it runs onesweep passes with tiles sorted in LDS first).
constexpr size_t kOwnSortMin = 393216, kOwnSortMax = 2097152;

struct SortLayout {
    size_t keys_out, vals_in, vals_out, temp, temp_bytes, total;
};

SortLayout sort_layout(size_t n) {
    SortLayout L{};
    size_t nn = n ? n : 1;
    size_t temp_bytes = 0;
    // size query only: no work is enqueued
    (void)rocprim::radix_sort_pairs(nullptr, temp_bytes, (const int32_t*)nullptr, (int32_t*)nullptr,
                                    (const uint32_t*)nullptr, (uint32_t*)nullptr, nn, 0u, 32u, (hipStream_t)0);
    size_t off = 0;
    L.keys_out = off; off = align_up(off + nn * 4, 256);
    L.vals_in = off;  off = align_up(off + nn * 4, 256);
    L.vals_out = off; off = align_up(off + nn * 4, 256);
    L.temp = off;     off = align_up(off + temp_bytes, 256);
    L.temp_bytes = temp_bytes;
    L.total = off;
    return L;
}

// counts[v * nblk + blk] = number of voxels of block blk whose mask has bit v set.  A block is kPairRows voxels, walked
// by kPairThreads threads in kPairRows / kPairThreads chunks.
__global__ void __launch_bounds__(kPairThreads) pair_count_kernel(const int32_t* __restrict__ gray, size_t n, int V,
                                                                  unsigned nblk, uint32_t* __restrict__ counts) {
    __shared__ uint32_t wave_cnt[kPairThreads / 64][32];
    constexpr int kChunks = kPairRows / kPairThreads;
    uint32_t g[kChunks];
#pragma unroll
    for (int c = 0; c < kChunks; ++c) {
        const size_t row = (size_t)blockIdx.x * kPairRows + c * kPairThreads + threadIdx.x;
        g[c] = row < n ? (uint32_t)gray[row] : 0u;
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (int v = 0; v < V; ++v) {
        uint32_t cnt = 0;
#pragma unroll
        for (int c = 0; c < kChunks; ++c) cnt += (uint32_t)__popcll(__ballot((g[c] >> v) & 1u));
        if (lane == 0) wave_cnt[wave][v] = cnt;
    }
    __syncthreads();
    if (threadIdx.x < V) {
        uint32_t c = 0;
        for (int w = 0; w < kPairThreads / 64; ++w) c += wave_cnt[w][threadIdx.x];
        counts[(size_t)threadIdx.x * nblk + blockIdx.x] = c;
    }
}

// seg[v] = offsets[v * nblk] for v < V, seg[V] = total (last offset + last count)
__global__ void pair_seg_kernel(const uint32_t* __restrict__ offsets, const uint32_t* __restrict__ counts, int V,
                                unsigned nblk, uint32_t* __restrict__ seg) {
    int v = threadIdx.x;
    if (v < V) seg[v] = nblk ? offsets[(size_t)v * nblk] : 0u;
    if (v == V) seg[V] = nblk ? offsets[(size_t)V * nblk - 1] + counts[(size_t)V * nblk - 1] : 0u;
}

// A block takes kPairRows voxels in chunks of kPairThreads: the chunk's map rows are staged in LDS with coalesced loads,
// then for every offset the present voxels are ranked (wave ballot + prefix of the wave totals) and (n, map[n, v]) goes
// to first[v] + rank, where first[v] starts at offsets[v, blk] and moves on by the chunk's count.  The pairs a block
// adds to one offset's list are therefore one run of up to kPairRows entries written by one workgroup within a few
// microseconds: the partial cache lines at the seams of the chunks' pieces meet in L2.
__global__ void __launch_bounds__(kPairThreads) pair_fill_kernel(const uint32_t* __restrict__ map,
                                                                 const int32_t* __restrict__ gray, size_t n, int V,
                                                                 unsigned nblk, const uint32_t* __restrict__ offsets,
                                                                 uint32_t* __restrict__ sig_i, uint32_t* __restrict__ sig_o) {
    extern __shared__ uint32_t lds[];
    constexpr int kWaves = kPairThreads / 64;
    uint32_t* rows = lds;                                    // [kPairThreads * V]
    uint32_t* wave_cnt2 = lds + (size_t)kPairThreads * V;    // [2][kWaves][32], by chunk parity
    uint32_t* first = wave_cnt2 + 2 * kWaves * 32;           // [32] where the next pairs of each offset go
    // fetched once, up front: a load inside the offset loop below would put a memory round trip into each of its turns
    if (threadIdx.x < V) first[threadIdx.x] = offsets[(size_t)threadIdx.x * nblk + blockIdx.x];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned long long below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    for (int c = 0; c < kPairRows / kPairThreads; ++c) {
        const size_t base = (size_t)blockIdx.x * kPairRows + (size_t)c * kPairThreads;
        if (base >= n) break;                                // uniform
        // two count tables: the first wavefront may still be adding up the previous chunk's counts (below) while the
        // others write this chunk's
        uint32_t* wave_cnt = wave_cnt2 + (c & 1) * kWaves * 32;
        const size_t len = (n - base < (size_t)kPairThreads ? n - base : (size_t)kPairThreads) * V;
        // eight loads in flight per thread: a plain copy loop waits for each load before it issues the next
        for (size_t i0 = 0; i0 < len; i0 += 8 * kPairThreads) {
            uint32_t t8[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const size_t i = i0 + (size_t)q * kPairThreads + threadIdx.x;
                t8[q] = i < len ? map[base * V + i] : 0u;
            }
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const size_t i = i0 + (size_t)q * kPairThreads + threadIdx.x;
                if (i < len) rows[i] = t8[q];
            }
        }
        const size_t row = base + threadIdx.x;
        const uint32_t g = row < n ? (uint32_t)gray[row] : 0u;
        for (int v = 0; v < V; ++v) {
            unsigned long long b = __ballot((g >> v) & 1u);
            if (lane == 0) wave_cnt[wave * 32 + v] = (uint32_t)__popcll(b);
        }
        __syncthreads();
        for (int v = 0; v < V; ++v) {
            unsigned long long b = __ballot((g >> v) & 1u);
            if ((g >> v) & 1u) {
                uint32_t r = (uint32_t)__popcll(b & below);
                for (int w = 0; w < wave; ++w) r += wave_cnt[w * 32 + v];
                size_t to = (size_t)first[v] + r;
                sig_o[to] = (uint32_t)row;
                sig_i[to] = rows[(size_t)threadIdx.x * V + v];
            }
        }
        __syncthreads();                                     // rows and first[] have been read by everyone
        if (threadIdx.x < V) {
            uint32_t add = 0;
            for (int w = 0; w < kWaves; ++w) add += wave_cnt[w * 32 + threadIdx.x];
            first[threadIdx.x] += add;
        }
        // the next chunk's first barrier orders these updates before they are read
    }
}

// One wavefront per tile: OR of gray[sorted_idx[r]] over the tile's rows.
__global__ void __launch_bounds__(kBlock) tile_or_kernel(const int32_t* __restrict__ gray,
                                                         const int64_t* __restrict__ sorted_idx, size_t n, int block,
                                                         size_t num_tiles, int32_t* __restrict__ tile_code,
                                                         uint32_t* __restrict__ popc) {
    const size_t tile = ((size_t)blockIdx.x * kBlock + threadIdx.x) >> 6;
    const int lane = threadIdx.x & 63;
    if (tile >= num_tiles) return;   // whole wavefronts leave together
    const size_t lo = tile * (size_t)block;
    const size_t hi = lo + (size_t)block < n ? lo + (size_t)block : n;
    uint32_t code = 0;
    for (size_t r = lo + lane; r < hi; r += 64) code |= (uint32_t)gray[sorted_idx[r]];
    for (int off = 32; off > 0; off >>= 1) code |= (uint32_t)__shfl_xor((int)code, off, 64);
    if (lane == 0) {
        tile_code[tile] = (int32_t)code;
        popc[tile] = (uint32_t)__popc(code);
    }
}

// seg[0..nb) = exclusive offsets (already there from the scan), seg[nb] = total
__global__ void tile_seg_tail_kernel(const uint32_t* __restrict__ popc, int32_t* __restrict__ seg, size_t num_tiles) {
    if (threadIdx.x == 0 && blockIdx.x == 0) seg[num_tiles] = seg[num_tiles - 1] + (int32_t)popc[num_tiles - 1];
}

__global__ void set_i32_kernel(int32_t* dst, int32_t value) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *dst = value;
}

__global__ void __launch_bounds__(kBlock) tile_fill_kernel(const int32_t* __restrict__ tile_code,
                                                           const int32_t* __restrict__ seg, size_t num_tiles,
                                                           int32_t* __restrict__ valid_kernel) {
    size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= num_tiles) return;
    uint32_t code = (uint32_t)tile_code[t];
    int32_t* dst = valid_kernel + seg[t];
    while (code) {
        *dst++ = __ffs((int)code) - 1;
        code &= code - 1;
    }
}

// Rows of the gather plan a tile contributes: one per offset present, and one (all rows missing) for a tile
// without any, so that every tile owns at least one step of the streaming GEMM.
__global__ void __launch_bounds__(kBlock) plan_count_kernel(const int32_t* __restrict__ tile_code, size_t num_tiles,
                                                            uint32_t* __restrict__ cnt) {
    size_t t = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (t >= num_tiles) return;
    const int c = __popc((uint32_t)tile_code[t]);
    cnt[t] = (uint32_t)(c > 0 ? c : 1);
}

// One workgroup per tile: plan_idx[seg[t] + k][r] = map[order[t * tile_rows + r]][k-th offset present in the tile]
// (EMPTY for rows past the end); plan_band[seg[t] + k] (optional) has bit b set when rows [32 b, 32 b + 32) of the
// tile hold at least one present neighbor for that offset.
__global__ void __launch_bounds__(kBlock) plan_fill_kernel(const uint32_t* __restrict__ map,
                                                           const int64_t* __restrict__ order,
                                                           const int32_t* __restrict__ tile_code,
                                                           const int32_t* __restrict__ seg, size_t n, int V, int tile_rows,
                                                           uint32_t* __restrict__ plan_idx, uint32_t* __restrict__ plan_band) {
    __shared__ uint32_t bands[32];
    __shared__ uint32_t stage[kBlock * 32];      // kBlock map rows of V <= 32 words
    __shared__ int64_t src_row[kBlock];          // which map row each of them is (-1: past the end)
    const size_t t = blockIdx.x;
    uint32_t code = (uint32_t)tile_code[t];
    size_t slot = (size_t)seg[t];
    if (code == 0) {
        for (int r = threadIdx.x; r < tile_rows; r += kBlock) plan_idx[slot * tile_rows + r] = FGX_EMPTY32;
        if (plan_band != nullptr && threadIdx.x == 0) plan_band[slot] = 0u;
        return;
    }
    if (threadIdx.x < 32) bands[threadIdx.x] = 0u;
    const int lane = threadIdx.x & 63;
    for (int r0 = 0; r0 < tile_rows; r0 += kBlock) {
        // The rows of this tile sit wherever the mask order put them.  A half-wave fetches one whole row (V consecutive
        // words: one or two cache lines per request) into LDS; each thread then walks its own row there.  One thread
        // per row reading straight from memory would ask for 64 different cache lines with every load instruction.
        __syncthreads();                         // the previous chunk's rows have been consumed; bands[] is cleared
        {
            const size_t row = t * (size_t)tile_rows + r0 + threadIdx.x;
            src_row[threadIdx.x] = (r0 + (int)threadIdx.x < tile_rows && row < n) ? order[row] : (int64_t)-1;
        }
        __syncthreads();
        for (int i0 = 0; i0 < kBlock * 32; i0 += 8 * kBlock) {       // eight loads in flight per thread
            uint32_t t8[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int i = i0 + q * kBlock + threadIdx.x;
                const int64_t src = src_row[i >> 5];
                t8[q] = ((i & 31) < V && src >= 0) ? map[(size_t)src * V + (i & 31)] : FGX_EMPTY32;
            }
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int i = i0 + q * kBlock + threadIdx.x;
                if ((i & 31) < V) stage[(i >> 5) * V + (i & 31)] = t8[q];
            }
        }
        __syncthreads();
        const int r = r0 + threadIdx.x;
        const uint32_t* mrow = src_row[threadIdx.x] >= 0 ? stage + threadIdx.x * V : nullptr;
        uint32_t c = code;
        size_t s = slot;
        int k = 0;
        while (c) {
            const int v = __ffs((int)c) - 1;
            c &= c - 1;
            const uint32_t m = mrow ? mrow[v] : FGX_EMPTY32;
            if (r < tile_rows) plan_idx[s * tile_rows + r] = m;
            if (plan_band != nullptr) {
                const unsigned long long live = __ballot(m != FGX_EMPTY32);    // all 64 lanes take part
                if (lane == 0) {
                    const int b0 = (r0 + (int)(threadIdx.x & ~63u)) >> 5;          // band of this wavefront's lanes 0-31
                    uint32_t bits = ((live & 0xFFFFFFFFull) ? 1u : 0u) << (b0 & 31);
                    bits |= ((live >> 32) ? 1u : 0u) << ((b0 + 1) & 31);
                    if (bits) atomicOr(&bands[k], bits);
                }
            }
            ++s;
            ++k;
        }
    }
    if (plan_band != nullptr) {
        __syncthreads();
        const int cnt = __popc(code);
        if ((int)threadIdx.x < cnt) plan_band[slot + threadIdx.x] = bands[threadIdx.x];
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Item order of the streaming GEMM (fgx_gather_item_order): one workgroup, no host round trip.
// ---------------------------------------------------------------------------------------------------------------
// Items (row tile * col_tiles + column tile) cost about max(popcount(tile_code), 1) offsets each.  Workgroup slot q of
// `groups` works through the positions q, q + groups, ... of the sequence written here.  Step 1 sorts the items by
// cost, most expensive first (stable counting sort over the 33 possible popcounts: per-thread counts of a contiguous
// chunk, one scan, one placement pass).  Step 2 deals them round by round: the incomplete last round takes the
// cheapest items, every full round gives its most expensive item to the least loaded slot (rank of each slot's load by
// counting).  Everything is deterministic.
constexpr int kOrderThreads = 1024;     // also the largest number of slots
constexpr int kCostBins = 33;

__global__ void __launch_bounds__(kOrderThreads) item_order_kernel(const int32_t* __restrict__ tile_code, unsigned num_tiles,
                                                                   unsigned col_tiles, unsigned slabs, unsigned groups,
                                                                   uint32_t* __restrict__ sorted, uint32_t* __restrict__ item_at) {
    __shared__ uint32_t count[kCostBins][kOrderThreads / 4];     // [bin][chunk owner]; 256 owners
    __shared__ uint32_t bin_start[kCostBins];
    __shared__ uint32_t load[kOrderThreads];
    constexpr unsigned kOwners = kOrderThreads / 4;
    const unsigned tid = threadIdx.x;
    const unsigned total = num_tiles * col_tiles;
    auto bin_of = [&](unsigned item) -> unsigned {                // bin 0 = most expensive
        const unsigned pc = (unsigned)__popc((uint32_t)tile_code[item / col_tiles]);
        return 32u - pc;
    };
    // ---- step 1: stable counting sort, cost descending ----
    for (unsigned i = tid; i < kCostBins * kOwners; i += kOrderThreads) (&count[0][0])[i] = 0u;
    __syncthreads();
    const unsigned chunk = (total + kOwners - 1) / kOwners;
    if (tid < kOwners) {
        const unsigned lo = tid * chunk, hi = lo + chunk < total ? lo + chunk : total;
        for (unsigned i = lo; i < hi; ++i) ++count[bin_of(i)][tid];
    }
    __syncthreads();
    if (tid < kCostBins) {                                        // per bin: exclusive prefix over the owners, total left in bin_start
        uint32_t run = 0;
        for (unsigned o = 0; o < kOwners; ++o) {
            const uint32_t c = count[tid][o];
            count[tid][o] = run;
            run += c;
        }
        bin_start[tid] = run;
    }
    __syncthreads();
    if (tid == 0) {
        uint32_t run = 0;
        for (int b = 0; b < kCostBins; ++b) {
            const uint32_t c = bin_start[b];
            bin_start[b] = run;
            run += c;
        }
    }
    __syncthreads();
    if (tid < kOwners) {
        const unsigned lo = tid * chunk, hi = lo + chunk < total ? lo + chunk : total;
        for (unsigned i = lo; i < hi; ++i) {
            const unsigned b = bin_of(i);
            sorted[bin_start[b] + count[b][tid]++] = i;
        }
    }
    __threadfence_block();
    __syncthreads();
    // ---- step 2: deal the rounds ----
    const unsigned rounds = total / groups, rem = total % groups;
    auto cost_of = [&](unsigned item) -> uint32_t {
        const unsigned pc = (unsigned)__popc((uint32_t)tile_code[item / col_tiles]);
        return (pc ? pc : 1u) * slabs + 3u;
    };
    uint32_t mine = 0;
    if (tid < rem) {                                              // cheapest items: the positions of the last round
        const unsigned item = sorted[total - rem + tid];
        item_at[rounds * groups + tid] = item;
        mine = cost_of(item);
    }
    for (unsigned r = 0; r < rounds; ++r) {
        if (tid < groups) load[tid] = mine;
        __syncthreads();
        if (tid < groups) {
            unsigned rank = 0;                                    // slots with a smaller load come first, ties by slot number
            for (unsigned q = 0; q < groups; ++q) {
                const uint32_t other = load[q];
                rank += (other < mine || (other == mine && q < tid)) ? 1u : 0u;
            }
            const unsigned item = sorted[r * groups + rank];      // rank 0 = least loaded slot <- most expensive item
            item_at[r * groups + tid] = item;
            mine += cost_of(item);
        }
        __syncthreads();
    }
}

size_t scan_temp_bytes(size_t count) {
    size_t bytes = 0;
    (void)rocprim::exclusive_scan(nullptr, bytes, (const uint32_t*)nullptr, (uint32_t*)nullptr, 0u, count ? count : 1,
                                  rocprim::plus<uint32_t>(), (hipStream_t)0);
    return bytes;
}

struct PairLayout {
    unsigned nblk;
    size_t counts, offsets, temp, temp_bytes, total;
};

PairLayout pair_layout(size_t n, int V) {
    PairLayout L{};
    L.nblk = cdiv(n, kPairRows);
    size_t cnt = (size_t)L.nblk * V;
    size_t off = 0;
    L.counts = off;  off = align_up(off + (cnt ? cnt : 1) * 4, 256);
    L.offsets = off; off = align_up(off + (cnt ? cnt : 1) * 4, 256);
    L.temp_bytes = scan_temp_bytes(cnt);
    L.temp = off;    off = align_up(off + L.temp_bytes, 256);
    L.total = off;
    return L;
}

struct TileLayout {
    size_t num_tiles, popc, temp, temp_bytes, total;
};

TileLayout tile_layout(size_t n, int block) {
    TileLayout L{};
    L.num_tiles = (n + block - 1) / block;
    size_t off = 0;
    L.popc = off; off = align_up(off + (L.num_tiles ? L.num_tiles : 1) * 4, 256);
    L.temp_bytes = scan_temp_bytes(L.num_tiles);
    L.temp = off; off = align_up(off + L.temp_bytes, 256);
    L.total = off;
    return L;
}

// rows ranked along the Z-order curve (batch index above 3 * bits interleaved coordinate bits) into ranked[]: a radix sort
// over the key bits a coordinate of the grid can differ in, on 32-bit keys when they fit
int zorder_rank(const int32_t* coords, size_t n, int bits_per_axis, int batch_bits, const LocalityLayout& L, char* ws,
                uint32_t* ranked, uint32_t* other, hipStream_t s, const char* what) {
    const unsigned grid = cdiv(n, kBlock);
    const unsigned end_bit = (unsigned)(3 * bits_per_axis + batch_bits);
    size_t temp_bytes = L.temp_bytes;
    if (end_bit <= 32) {
        uint32_t* keys_a = (uint32_t*)(ws + L.keys_a);
        uint32_t* keys_b = (uint32_t*)(ws + L.keys_b);
        morton_key_packed_kernel<uint32_t><<<grid, kBlock, 0, s>>>(coords, n, bits_per_axis, keys_a, other);
        FGX_CHECK_LAUNCH(what);
        FGX_CHECK_HIP(rocprim::radix_sort_pairs(ws + L.temp, temp_bytes, keys_a, keys_b, other, ranked, n, 0u, end_bit, s));
    } else {
        uint64_t* keys_a = (uint64_t*)(ws + L.keys_a);
        uint64_t* keys_b = (uint64_t*)(ws + L.keys_b);
        morton_key_packed_kernel<uint64_t><<<grid, kBlock, 0, s>>>(coords, n, bits_per_axis, keys_a, other);
        FGX_CHECK_LAUNCH(what);
        FGX_CHECK_HIP(rocprim::radix_sort_pairs(ws + L.temp, temp_bytes, keys_a, keys_b, other, ranked, n, 0u, end_bit, s));
    }
    return FGX_OK;
}


}  // namespace
}  // namespace fgx

using namespace fgx;

extern "C" {

size_t fgx_sort_workspace_bytes(size_t n) {
    // (in the radix sort's range a call with a full 32-bit code still takes the library sort: room for either)
    const size_t lib_sort = sort_layout(n).total;
    if (n < kOwnSortMin || n > kOwnSortMax) return lib_sort;
    const size_t own = radix_layout(n).total;
    return own > lib_sort ? own : lib_sort;
}

int fgx_sort_by_code(const int32_t* binary, size_t n, int V, int64_t* sorted_idx, void* workspace,
                     size_t workspace_bytes, fgx_stream_t stream) {
    FGX_CHECK_ARG(V >= 1 && V <= 32, "fgx_sort_by_code: kernel volume must be in [1, 32], got %d", V);
    FGX_CHECK_ARG(n < 0xFFFFFFFFull, "fgx_sort_by_code: too many rows");
    if (n == 0) return FGX_OK;
    const bool own = n >= kOwnSortMin && n <= kOwnSortMax;
    const size_t need = fgx_sort_workspace_bytes(n);
    FGX_CHECK_ARG(binary && sorted_idx && workspace, "fgx_sort_by_code: null buffer");
    FGX_CHECK_ARG(workspace_bytes >= need, "fgx_sort_by_code: workspace of %zu bytes, need %zu", workspace_bytes, need);
    FGX_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fgx_sort_by_code: workspace must be 256-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)workspace;
    PhaseEnd phases{s};
    phase_mark("mask sort", s);
    // With V < 32 every key is non-negative and only bits [0, V) can differ.
    const unsigned end_bit = V < 32 ? (unsigned)V : 32u;
    if (own && V < 32) {
        // (as unsigned numbers the keys then order like the int32 codes); the first pass numbers the rows itself and the
        // last one writes the 64-bit indices
        return radix_sort_pairs_u32((const uint32_t*)binary, nullptr, n, end_bit, ws, radix_layout(n), nullptr, nullptr, sorted_idx, s,
                                    "fgx_sort_by_code");
    }
    const SortLayout L = sort_layout(n);
    int32_t* keys_out = (int32_t*)(ws + L.keys_out);
    uint32_t* vals_in = (uint32_t*)(ws + L.vals_in);
    uint32_t* vals_out = (uint32_t*)(ws + L.vals_out);
    iota_u32_kernel<<<cdiv(n, kBlock), kBlock, 0, s>>>(vals_in, n);
    FGX_CHECK_LAUNCH("fgx_sort_by_code(iota)");
    size_t temp_bytes = L.temp_bytes;
    FGX_CHECK_HIP(rocprim::radix_sort_pairs(ws + L.temp, temp_bytes, binary, keys_out, vals_in, vals_out, n, 0u, end_bit, s));
    widen_u32_i64_kernel<<<cdiv(n, kBlock), kBlock, 0, s>>>(vals_out, sorted_idx, n);
    FGX_CHECK_LAUNCH("fgx_sort_by_code(widen)");
    return FGX_OK;
}

size_t fgx_locality_workspace_bytes(size_t n) { return locality_layout(n).total; }

int fgx_locality_order_grid(const int32_t* coords, const int32_t* binary, size_t n, int V, int chunk_rows, int bits_per_axis,
                            int batch_bits, int64_t* order, void* workspace, size_t workspace_bytes, fgx_stream_t stream) {
    FGX_CHECK_ARG(V >= 1 && V <= 32, "fgx_locality_order: kernel volume must be in [1, 32], got %d", V);
    FGX_CHECK_ARG(chunk_rows >= 1, "fgx_locality_order: chunk_rows must be positive, got %d", chunk_rows);
    FGX_CHECK_ARG(bits_per_axis >= 1 && bits_per_axis <= 16 && batch_bits >= 0 && 3 * bits_per_axis + batch_bits <= 64,
                  "fgx_locality_order: %d bits per axis and %d batch bits do not fit a 64-bit key", bits_per_axis, batch_bits);
    FGX_CHECK_ARG(n < 0xFFFFFFFFull, "fgx_locality_order: too many rows");
    if (n == 0) return FGX_OK;
    LocalityLayout L = locality_layout(n);
    FGX_CHECK_ARG(coords && binary && order && workspace, "fgx_locality_order: null buffer");
    FGX_CHECK_ARG(((uintptr_t)coords & 15) == 0, "fgx_locality_order: coords must be 16-byte aligned");
    FGX_CHECK_ARG(workspace_bytes >= L.total, "fgx_locality_order: workspace of %zu bytes, need %zu", workspace_bytes, L.total);
    FGX_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fgx_locality_order: workspace must be 256-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)workspace;
    uint64_t* keys_a = (uint64_t*)(ws + L.keys_a);
    uint64_t* keys_b = (uint64_t*)(ws + L.keys_b);
    uint32_t* vals_a = (uint32_t*)(ws + L.vals_a);
    uint32_t* vals_b = (uint32_t*)(ws + L.vals_b);
    const unsigned grid = cdiv(n, kBlock);
    int rc = zorder_rank(coords, n, bits_per_axis, batch_bits, L, ws, vals_b, vals_a, s, "fgx_locality_order(keys)");
    if (rc != FGX_OK) return rc;
    if (chunk_rows == 1) {              // chunks of one rank: the curve's own order, nothing to sort inside them
        widen_u32_i64_kernel<<<grid, kBlock, 0, s>>>(vals_b, order, n);
        FGX_CHECK_LAUNCH("fgx_locality_order(widen)");
        return FGX_OK;
    }
    // (chunk, mask code) keys with the chunk right above the V code bits: the sort runs over the bits in use alone
    chunk_code_key_kernel<<<grid, kBlock, 0, s>>>(vals_b, binary, n, (uint32_t)chunk_rows, V, keys_a);
    FGX_CHECK_LAUNCH("fgx_locality_order(chunk keys)");
    const unsigned end_bit = (unsigned)V + (unsigned)bits_for((n - 1) / (size_t)chunk_rows);
    size_t temp_bytes = L.temp_bytes;
    FGX_CHECK_HIP(rocprim::radix_sort_pairs(ws + L.temp, temp_bytes, keys_a, keys_b, vals_b, vals_a, n, 0u, end_bit, s));
    widen_u32_i64_kernel<<<grid, kBlock, 0, s>>>(vals_a, order, n);
    FGX_CHECK_LAUNCH("fgx_locality_order(widen)");
    return FGX_OK;
}

int fgx_locality_order(const int32_t* coords, const int32_t* binary, size_t n, int V, int chunk_rows, int64_t* order,
                       void* workspace, size_t workspace_bytes, fgx_stream_t stream) {
    // coordinates of any grid: 16 bits per axis and 16 bits of batch index
    return fgx_locality_order_grid(coords, binary, n, V, chunk_rows, 16, 16, order, workspace, workspace_bytes, stream);
}

int fgx_zorder_rows(const int32_t* coords, size_t n, int bits_per_axis, int batch_bits, int64_t* order, void* workspace,
                    size_t workspace_bytes, fgx_stream_t stream) {
    FGX_CHECK_ARG(bits_per_axis >= 1 && bits_per_axis <= 16 && batch_bits >= 0 && 3 * bits_per_axis + batch_bits <= 64,
                  "fgx_zorder_rows: %d bits per axis and %d batch bits do not fit a 64-bit key", bits_per_axis, batch_bits);
    FGX_CHECK_ARG(n < 0xFFFFFFFFull, "fgx_zorder_rows: too many rows");
    if (n == 0) return FGX_OK;
    LocalityLayout L = locality_layout(n);
    FGX_CHECK_ARG(coords && order && workspace, "fgx_zorder_rows: null buffer");
    FGX_CHECK_ARG(((uintptr_t)coords & 15) == 0, "fgx_zorder_rows: coords must be 16-byte aligned");
    FGX_CHECK_ARG(workspace_bytes >= L.total, "fgx_zorder_rows: workspace of %zu bytes, need %zu", workspace_bytes, L.total);
    FGX_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fgx_zorder_rows: workspace must be 256-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)workspace;
    uint32_t* vals_a = (uint32_t*)(ws + L.vals_a);
    uint32_t* vals_b = (uint32_t*)(ws + L.vals_b);
    int rc = zorder_rank(coords, n, bits_per_axis, batch_bits, L, ws, vals_b, vals_a, s, "fgx_zorder_rows(keys)");
    if (rc != FGX_OK) return rc;
    widen_u32_i64_kernel<<<cdiv(n, kBlock), kBlock, 0, s>>>(vals_b, order, n);
    FGX_CHECK_LAUNCH("fgx_zorder_rows(widen)");
    return FGX_OK;
}

size_t fgx_pair_workspace_bytes(size_t n, int V) { return pair_layout(n, V > 0 ? V : 1).total; }

int fgx_pair_count(const int32_t* gray, size_t n, int V, uint32_t* seg, void* workspace, size_t workspace_bytes,
                   fgx_stream_t stream) {
    FGX_CHECK_ARG(V >= 1 && V <= 32, "fgx_pair_count: kernel volume must be in [1, 32], got %d", V);
    FGX_CHECK_ARG(seg != nullptr, "fgx_pair_count: null segment table");
    FGX_CHECK_ARG(n * (size_t)V < 0xFFFFFFFFull, "fgx_pair_count: pair offsets must fit in 32 bits");
    hipStream_t s = (hipStream_t)stream;
    PairLayout L = pair_layout(n, V);
    if (n > 0) {
        FGX_CHECK_ARG(gray && workspace, "fgx_pair_count: null buffer");
        FGX_CHECK_ARG(workspace_bytes >= L.total, "fgx_pair_count: workspace of %zu bytes, need %zu", workspace_bytes, L.total);
        FGX_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fgx_pair_count: workspace must be 256-byte aligned");
    }
    char* ws = (char*)workspace;
    uint32_t* counts = n ? (uint32_t*)(ws + L.counts) : nullptr;
    uint32_t* offsets = n ? (uint32_t*)(ws + L.offsets) : nullptr;
    PhaseEnd phases{s};
    phase_mark("pair count", s);
    if (n > 0) {
        pair_count_kernel<<<L.nblk, kPairThreads, 0, s>>>(gray, n, V, L.nblk, counts);
        FGX_CHECK_LAUNCH("fgx_pair_count(count)");
        size_t temp_bytes = L.temp_bytes;
        FGX_CHECK_HIP(rocprim::exclusive_scan(ws + L.temp, temp_bytes, counts, offsets, 0u, (size_t)L.nblk * V,
                                              rocprim::plus<uint32_t>(), s));
    }
    pair_seg_kernel<<<1, 64, 0, s>>>(offsets, counts, V, n ? L.nblk : 0u, seg);
    FGX_CHECK_LAUNCH("fgx_pair_count(seg)");
    return FGX_OK;
}

int fgx_pair_fill(const uint32_t* map, const int32_t* gray, size_t n, int V, const void* workspace, uint32_t* sig_i,
                  uint32_t* sig_o, fgx_stream_t stream) {
    FGX_CHECK_ARG(V >= 1 && V <= 32, "fgx_pair_fill: kernel volume must be in [1, 32], got %d", V);
    if (n == 0) return FGX_OK;
    FGX_CHECK_ARG(map && gray && workspace && sig_i && sig_o, "fgx_pair_fill: null buffer");
    PairLayout L = pair_layout(n, V);
    const uint32_t* offsets = (const uint32_t*)((const char*)workspace + L.offsets);
    size_t lds = ((size_t)kPairThreads * V + 2 * (kPairThreads / 64) * 32 + 32) * sizeof(uint32_t);
    PhaseEnd phases{(hipStream_t)stream};
    phase_mark("pair fill", (hipStream_t)stream);
    pair_fill_kernel<<<L.nblk, kPairThreads, lds, (hipStream_t)stream>>>(map, gray, n, V, L.nblk, offsets, sig_i, sig_o);
    FGX_CHECK_LAUNCH("fgx_pair_fill");
    return FGX_OK;
}

size_t fgx_tile_workspace_bytes(size_t n, int block) { return tile_layout(n, block > 0 ? block : 1).total; }

int fgx_tile_codes(const int32_t* gray, const int64_t* sorted_idx, size_t n, int block, int32_t* tile_code,
                   int32_t* seg, void* workspace, size_t workspace_bytes, fgx_stream_t stream) {
    FGX_CHECK_ARG(block >= 1, "fgx_tile_codes: tile size must be >= 1, got %d", block);
    FGX_CHECK_ARG(seg != nullptr, "fgx_tile_codes: null segment table");
    hipStream_t s = (hipStream_t)stream;
    TileLayout L = tile_layout(n, block);
    if (L.num_tiles == 0) {
        set_i32_kernel<<<1, 64, 0, s>>>(seg, 0);
        FGX_CHECK_LAUNCH("fgx_tile_codes(empty)");
        return FGX_OK;
    }
    FGX_CHECK_ARG(gray && sorted_idx && tile_code && workspace, "fgx_tile_codes: null buffer");
    FGX_CHECK_ARG(workspace_bytes >= L.total, "fgx_tile_codes: workspace of %zu bytes, need %zu", workspace_bytes, L.total);
    FGX_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fgx_tile_codes: workspace must be 256-byte aligned");
    char* ws = (char*)workspace;
    uint32_t* popc = (uint32_t*)(ws + L.popc);
    PhaseEnd phases{s};
    phase_mark("tile masks", s);
    tile_or_kernel<<<cdiv(L.num_tiles * 64, kBlock), kBlock, 0, s>>>(gray, sorted_idx, n, block, L.num_tiles, tile_code, popc);
    FGX_CHECK_LAUNCH("fgx_tile_codes(or)");
    size_t temp_bytes = L.temp_bytes;
    FGX_CHECK_HIP(rocprim::exclusive_scan(ws + L.temp, temp_bytes, popc, (uint32_t*)seg, 0u, L.num_tiles,
                                          rocprim::plus<uint32_t>(), s));
    tile_seg_tail_kernel<<<1, 64, 0, s>>>(popc, seg, L.num_tiles);
    FGX_CHECK_LAUNCH("fgx_tile_codes(tail)");
    return FGX_OK;
}

int fgx_tile_fill(const int32_t* tile_code, const int32_t* seg, size_t num_tiles, int32_t* valid_kernel,
                  fgx_stream_t stream) {
    if (num_tiles == 0) return FGX_OK;
    FGX_CHECK_ARG(tile_code && seg && valid_kernel, "fgx_tile_fill: null buffer");
    tile_fill_kernel<<<cdiv(num_tiles, kBlock), kBlock, 0, (hipStream_t)stream>>>(tile_code, seg, num_tiles, valid_kernel);
    FGX_CHECK_LAUNCH("fgx_tile_fill");
    return FGX_OK;
}

int fgx_gather_plan_count(const int32_t* tile_code, size_t num_tiles, int32_t* plan_seg, void* workspace,
                          size_t workspace_bytes, fgx_stream_t stream) {
    FGX_CHECK_ARG(plan_seg != nullptr, "fgx_gather_plan_count: null segment table");
    hipStream_t s = (hipStream_t)stream;
    if (num_tiles == 0) {
        set_i32_kernel<<<1, 64, 0, s>>>(plan_seg, 0);
        FGX_CHECK_LAUNCH("fgx_gather_plan_count(empty)");
        return FGX_OK;
    }
    TileLayout L = tile_layout(num_tiles, 1);
    FGX_CHECK_ARG(tile_code && workspace, "fgx_gather_plan_count: null buffer");
    FGX_CHECK_ARG(workspace_bytes >= L.total, "fgx_gather_plan_count: workspace of %zu bytes, need %zu", workspace_bytes, L.total);
    FGX_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fgx_gather_plan_count: workspace must be 256-byte aligned");
    unsigned char* ws = (unsigned char*)workspace;
    uint32_t* cnt = (uint32_t*)(ws + L.popc);
    PhaseEnd phases{s};
    phase_mark("gather plan count", s);
    plan_count_kernel<<<cdiv(num_tiles, kBlock), kBlock, 0, s>>>(tile_code, num_tiles, cnt);
    FGX_CHECK_LAUNCH("fgx_gather_plan_count(count)");
    size_t temp_bytes = L.temp_bytes;
    FGX_CHECK_HIP(rocprim::exclusive_scan(ws + L.temp, temp_bytes, cnt, (uint32_t*)plan_seg, 0u, num_tiles,
                                          rocprim::plus<uint32_t>(), s));
    tile_seg_tail_kernel<<<1, 64, 0, s>>>(cnt, plan_seg, num_tiles);
    FGX_CHECK_LAUNCH("fgx_gather_plan_count(tail)");
    return FGX_OK;
}

int fgx_gather_plan_fill(const uint32_t* map, const int64_t* order, const int32_t* tile_code, const int32_t* plan_seg,
                         size_t n, int V, int tile_rows, uint32_t* plan_idx, uint32_t* plan_band, fgx_stream_t stream) {
    FGX_CHECK_ARG(tile_rows >= 1 && V >= 1 && V <= 32, "fgx_gather_plan_fill: bad shape tile_rows=%d V=%d", tile_rows, V);
    if (n == 0) return FGX_OK;
    FGX_CHECK_ARG(map && order && tile_code && plan_seg && plan_idx, "fgx_gather_plan_fill: null buffer");
    const size_t num_tiles = (n + tile_rows - 1) / tile_rows;
    FGX_CHECK_ARG(num_tiles <= 0x7FFFFFFFu, "fgx_gather_plan_fill: too many tiles");
    FGX_CHECK_ARG(plan_band == nullptr || tile_rows <= 1024, "fgx_gather_plan_fill: band masks need tile_rows <= 1024");
    PhaseEnd phases{(hipStream_t)stream};
    phase_mark("gather plan fill", (hipStream_t)stream);
    plan_fill_kernel<<<(unsigned)num_tiles, kBlock, 0, (hipStream_t)stream>>>(map, order, tile_code, plan_seg, n, V, tile_rows,
                                                                              plan_idx, plan_band);
    FGX_CHECK_LAUNCH("fgx_gather_plan_fill");
    return FGX_OK;
}

size_t fgx_gather_item_order_workspace_bytes(size_t num_tiles, int col_tiles) {
    if (col_tiles < 1) return 0;
    return align_up((num_tiles * (size_t)col_tiles + 1) * sizeof(uint32_t), 256);
}

int fgx_gather_item_order(const int32_t* tile_code, size_t num_tiles, int col_tiles, int slabs, int groups, void* workspace,
                          size_t workspace_bytes, uint32_t* item_at, fgx_stream_t stream) {
    FGX_CHECK_ARG(col_tiles >= 1 && slabs >= 1, "fgx_gather_item_order: bad shape col_tiles=%d slabs=%d", col_tiles, slabs);
    FGX_CHECK_ARG(groups >= 1 && groups <= kOrderThreads, "fgx_gather_item_order: groups must be in [1, %d], got %d", kOrderThreads,
                  groups);
    const size_t total = num_tiles * (size_t)col_tiles;
    if (total == 0) return FGX_OK;
    FGX_CHECK_ARG(total < 0x7FFFFFFFull, "fgx_gather_item_order: too many items");
    FGX_CHECK_ARG(tile_code && workspace && item_at, "fgx_gather_item_order: null buffer");
    FGX_CHECK_ARG(workspace_bytes >= fgx_gather_item_order_workspace_bytes(num_tiles, col_tiles),
                  "fgx_gather_item_order: workspace of %zu bytes is too small", workspace_bytes);
    FGX_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fgx_gather_item_order: workspace must be 256-byte aligned");
    item_order_kernel<<<1, kOrderThreads, 0, (hipStream_t)stream>>>(tile_code, (unsigned)num_tiles, (unsigned)col_tiles,
                                                                    (unsigned)slabs, (unsigned)groups, (uint32_t*)workspace, item_at);
    FGX_CHECK_LAUNCH("fgx_gather_item_order");
    return FGX_OK;
}

}  // extern "C"
