// Stable LSD radix sort of (32-bit key, row index) pairs for gfx950, for the sorts of the neighbor-cache build:
// a few hundred thousand to a few million items whose keys have 20 ... 32 significant bits.
//
// Below about a million items the library sort runs a ladder of ~20 small merge kernels (0.13 ms for 669 288 items),
// above it four onesweep passes.  Here every pass is three launches over digits of up to 10 bits (27-bit mask keys:
// three passes): a histogram per tile of 1024 items, an exclusive scan over the [digit][tile] table (one workgroup per
// digit scans its row of tiles and leaves the row's total; the scatter adds the totals of the lower digits), and a scatter in
// which one wavefront walks its tile 64 items at a time -- the lanes holding the same digit find each other with one
// ballot per digit bit, the lowest of them takes the run's place from a per-digit counter in LDS -- so equal digits
// keep their order (stable) without any cross-wavefront ordering.  The first pass can take the row index from the
// item's position, the last pass can write 64-bit indices and drop the keys.
#pragma once
#include "fgx_common.h"

namespace fgx {
namespace {

constexpr int kRsRounds = 16;        // a wavefront takes its tile 64 items at a time
constexpr int kRsTile = 64 * kRsRounds;   // items per tile (one wavefront each)
constexpr int kRsMaxBits = 10;       // digit width limit: 1024 counters of LDS per wavefront

constexpr unsigned kRsMaxTiles = 256 * 16;   // tiles a digit's row may have: one workgroup scans it, 16 entries per thread

struct RadixLayout {
    unsigned tiles;
    size_t keys_a, keys_b, vals_a, vals_b, hist, offs, totals, total;
};

inline RadixLayout radix_layout(size_t n) {
    RadixLayout L{};
    const size_t nn = n ? n : 1;
    L.tiles = cdiv(nn, (size_t)kRsTile);
    size_t off = 0;
    L.keys_a = off;
    off = align_up(off + nn * 4, 256);
    L.keys_b = off;
    off = align_up(off + nn * 4, 256);
    L.vals_a = off;
    off = align_up(off + nn * 4, 256);
    L.vals_b = off;
    off = align_up(off + nn * 4, 256);
    L.hist = off;
    const size_t entries = ((size_t)1 << kRsMaxBits) * L.tiles;
    off = align_up(off + entries * 4, 256);
    L.offs = off;
    off = align_up(off + entries * 4, 256);
    L.totals = off;
    off = align_up(off + ((size_t)1 << kRsMaxBits) * 4, 256);
    L.total = off;
    return L;
}

// hist[digit * tiles + tile] = items of the tile with that digit.  run_if != nullptr: the whole sort is conditional on that
// word, which an earlier kernel of the stream has written -- every wavefront returns at once when it is zero.
__global__ void __launch_bounds__(64) radix_hist_kernel(const uint32_t* __restrict__ keys, size_t n, unsigned shift, unsigned bits,
                                                        unsigned tiles, uint32_t* __restrict__ hist,
                                                        const uint32_t* __restrict__ run_if) {
    if (run_if != nullptr && *run_if == 0u) return;
    __shared__ uint32_t count[1 << kRsMaxBits];
    const unsigned bins = 1u << bits, mask = bins - 1u;
    for (unsigned b = threadIdx.x; b < bins; b += 64) count[b] = 0u;
    __syncthreads();
    const size_t base = (size_t)blockIdx.x * kRsTile;
    uint32_t key[kRsRounds];
#pragma unroll
    for (int r = 0; r < kRsRounds; ++r) {           // all loads of the tile in flight together
        const size_t i = base + (size_t)r * 64 + threadIdx.x;
        key[r] = i < n ? keys[i] : 0u;
    }
#pragma unroll
    for (int r = 0; r < kRsRounds; ++r) {
        const size_t i = base + (size_t)r * 64 + threadIdx.x;
        if (i < n) atomicAdd(&count[(key[r] >> shift) & mask], 1u);
    }
    __syncthreads();
    for (unsigned b = threadIdx.x; b < bins; b += 64) hist[(size_t)b * tiles + blockIdx.x] = count[b];
}

// offs[digit][tile] = items with that digit in the tiles before this one; totals[digit] = items with that digit.  One
// workgroup per digit: a thread adds up 16 consecutive tiles, the 256 sums are scanned through LDS, the thread writes its
// 16 prefixes.
__global__ void __launch_bounds__(256) radix_row_scan_kernel(const uint32_t* __restrict__ hist, unsigned tiles,
                                                             uint32_t* __restrict__ offs, uint32_t* __restrict__ totals,
                                                             const uint32_t* __restrict__ run_if) {
    if (run_if != nullptr && *run_if == 0u) return;
    __shared__ uint32_t part[256];
    const uint32_t* row = hist + (size_t)blockIdx.x * tiles;
    uint32_t* out = offs + (size_t)blockIdx.x * tiles;
    const unsigned per = (tiles + 255u) / 256u;         // consecutive tiles per thread (at most 16)
    const unsigned t0 = threadIdx.x * per;
    uint32_t v[16];
    uint32_t sum = 0u;
#pragma unroll
    for (unsigned k = 0; k < 16; ++k) {
        v[k] = (k < per && t0 + k < tiles) ? row[t0 + k] : 0u;
        sum += v[k];
    }
    part[threadIdx.x] = sum;
    __syncthreads();
    for (unsigned d = 1; d < 256; d <<= 1) {            // inclusive scan of the 256 sums
        const uint32_t add = threadIdx.x >= d ? part[threadIdx.x - d] : 0u;
        __syncthreads();
        part[threadIdx.x] += add;
        __syncthreads();
    }
    uint32_t run = part[threadIdx.x] - sum;
#pragma unroll
    for (unsigned k = 0; k < 16; ++k) {
        if (k < per && t0 + k < tiles) out[t0 + k] = run;
        run += v[k];
    }
    if (threadIdx.x == 255) totals[blockIdx.x] = part[255];
}

// Item i of the tile goes to (items with a lower digit) + offs[digit][tile] + (items of the tile with the same
// digit before it).  vals_in == nullptr: the value is the item's position.  out64 != nullptr: last pass, the values are
// written there as 64-bit integers and neither keys nor 32-bit values are written.
__global__ void __launch_bounds__(64) radix_scatter_kernel(const uint32_t* __restrict__ keys, const uint32_t* __restrict__ vals_in,
                                                           size_t n, unsigned shift, unsigned bits, unsigned tiles,
                                                           const uint32_t* __restrict__ offs, const uint32_t* __restrict__ totals,
                                                           uint32_t* __restrict__ keys_out,
                                                           uint32_t* __restrict__ vals_out, int64_t* __restrict__ out64,
                                                           const uint32_t* __restrict__ run_if) {
    if (run_if != nullptr && *run_if == 0u) return;
    __shared__ uint32_t next[1 << kRsMaxBits];        // where the next item of each digit goes
    const unsigned bins = 1u << bits, mask = bins - 1u;
    const unsigned lane = threadIdx.x;
    {
        // items with a lower digit: an exclusive scan of the digit totals, 16 consecutive digits per lane
        const unsigned per = (bins + 63u) / 64u;
        uint32_t tv[16];
        uint32_t sum = 0u;
#pragma unroll
        for (unsigned k = 0; k < 16; ++k) {
            tv[k] = (k < per && lane * per + k < bins) ? totals[lane * per + k] : 0u;
            sum += tv[k];
        }
        uint32_t incl = sum;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t o = (uint32_t)__shfl_up((int)incl, d, 64);
            if ((int)lane >= d) incl += o;
        }
        uint32_t run = incl - sum;
#pragma unroll
        for (unsigned k = 0; k < 16; ++k) {
            const unsigned b = lane * per + k;
            if (k < per && b < bins) next[b] = run + offs[(size_t)b * tiles + blockIdx.x];
            run += tv[k];
        }
    }
    __syncthreads();
    const size_t base = (size_t)blockIdx.x * kRsTile;
    const unsigned long long below = (1ull << lane) - 1ull;
    uint32_t key_r[kRsRounds], val_r[kRsRounds];
#pragma unroll
    for (int r = 0; r < kRsRounds; ++r) {           // all loads of the tile in flight together
        const size_t i = base + (size_t)r * 64 + lane;
        key_r[r] = i < n ? keys[i] : 0u;
        val_r[r] = i < n ? (vals_in ? vals_in[i] : (uint32_t)i) : 0u;
    }
#pragma unroll
    for (int r = 0; r < kRsRounds; ++r) {
        const size_t i = base + (size_t)r * 64 + lane;
        const bool live = i < n;
        const uint32_t key = key_r[r], val = val_r[r];
        const uint32_t digit = (key >> shift) & mask;
        unsigned long long peers = __ballot(live);
        for (unsigned b = 0; b < bits; ++b) {
            const bool bit = (digit >> b) & 1u;
            const unsigned long long have = __ballot(bit);
            peers &= bit ? have : ~have;
        }
        // the lowest lane of a run of equal digits takes the run's place; one wavefront, so LDS accesses stay in order
        uint32_t first = 0u;
        const int leader = live ? __ffsll((long long)peers) - 1 : 0;
        if (live && (int)lane == leader) {
            first = next[digit];
            next[digit] = first + (uint32_t)__popcll(peers);
        }
        first = __shfl(first, leader, 64);
        if (live) {
            const size_t pos = (size_t)first + (size_t)__popcll(peers & below);
            if (out64) {
                out64[pos] = (int64_t)val;
            } else {
                keys_out[pos] = key;
                vals_out[pos] = val;
            }
        }
    }
}

// Sorts (keys[i], vals[i] or i) by the low `end_bit` bits of the keys, stable.  `ws`: radix_layout(n).total bytes, 256-byte
// aligned.  The result ends in (*keys_sorted, *vals_sorted), which point into the workspace, or, with out64, in out64 alone.
// run_if (a device word, or nullptr): when it reads zero every kernel of the sort returns at once and the buffers the result
// would have ended in are left as they were.
inline int radix_sort_pairs_u32(const uint32_t* keys, const uint32_t* vals, size_t n, unsigned end_bit, char* ws, const RadixLayout& L,
                                const uint32_t** keys_sorted, const uint32_t** vals_sorted, int64_t* out64, hipStream_t s,
                                const char* what, const uint32_t* run_if = nullptr) {
    if (end_bit < 1) end_bit = 1;
    if (end_bit > 32) end_bit = 32;
    const unsigned passes = (end_bit + kRsMaxBits - 1) / kRsMaxBits;
    const unsigned bits = (end_bit + passes - 1) / passes;
    uint32_t* kbuf[2] = {(uint32_t*)(ws + L.keys_a), (uint32_t*)(ws + L.keys_b)};
    uint32_t* vbuf[2] = {(uint32_t*)(ws + L.vals_a), (uint32_t*)(ws + L.vals_b)};
    uint32_t* hist = (uint32_t*)(ws + L.hist);
    uint32_t* offs = (uint32_t*)(ws + L.offs);
    uint32_t* totals = (uint32_t*)(ws + L.totals);
    if (L.tiles > kRsMaxTiles) {
        set_error("%s: %zu items are more than the radix sort's table scan takes", what, n);
        return FGX_ERR_UNSUPPORTED;
    }
    const uint32_t* kin = keys;
    const uint32_t* vin = vals;
    for (unsigned p = 0; p < passes; ++p) {
        const unsigned shift = p * bits;
        const bool last = p + 1 == passes;
        radix_hist_kernel<<<L.tiles, 64, 0, s>>>(kin, n, shift, bits, L.tiles, hist, run_if);
        FGX_CHECK_LAUNCH(what);
        radix_row_scan_kernel<<<1u << bits, 256, 0, s>>>(hist, L.tiles, offs, totals, run_if);
        FGX_CHECK_LAUNCH(what);
        radix_scatter_kernel<<<L.tiles, 64, 0, s>>>(kin, vin, n, shift, bits, L.tiles, offs, totals, kbuf[p & 1], vbuf[p & 1],
                                                    last ? out64 : nullptr, run_if);
        FGX_CHECK_LAUNCH(what);
        kin = kbuf[p & 1];
        vin = vbuf[p & 1];
    }
    if (keys_sorted) *keys_sorted = kin;
    if (vals_sorted) *vals_sorted = vin;
    return FGX_OK;
}

}  // namespace
}  // namespace fgx
