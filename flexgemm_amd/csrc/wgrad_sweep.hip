// Weight gradient of the masked implicit GEMM as a sweep over the voxels, for gfx950 (16-bit types, a single Co x Ci
// tile of 128 x 128 or 64 x 64, up to 2^24 voxels).
//
// grad_weight[:, v, :] = sum over the pairs (n -> m at offset v) of grad_out[n]^T feats[m]
// (reference: flex_gemm/kernels/triton/spconv/sparse_submanifold_conv_bwd_masked_implicit_gemm_splitk.py:108-182,
// 278-317, which cuts the pairs of every offset into SPLITK slices with a partial product each).
//
// The block-major kernel of wgrad_gemm.hip cuts the voxels into blocks of ~12K rows and writes an fp32 partial product
// per (block, offset).  Here
//
//   * XCD x owns a contiguous range of sub-blocks holding an eighth of the pairs (pair lists ascend in the output row
//     inside every offset, so that is one contiguous pair range per offset);
//   * every offset is cut into up to 64 slices that take its 64-pair steps in turn, a unit is a set of slices of one
//     offset, and every workgroup gets at most two units of together (nearly) the same number of steps and KEEPS BOTH
//     ACCUMULATORS IN REGISTERS for the whole range: 512 partial products in all instead of one per (block, offset);
//   * a workgroup takes the steps of its two units in the order of the sub-blocks their pairs lie in, changing units
//     every ~16K voxels.  Loaders and multipliers meet through progress words in LDS, not at a barrier per step: a
//     loader owns a ring stage and whole steps, a multiplier's fragment reads run on across the end of a step;
//   * the bias gradient (column sums of grad_out over the offset whose pairs hold every output row once) is added up
//     by the loaders from what they deposited in their stages;
//   * optionally the workgroups of an XCD pace each other: nobody starts a sub-block more than `lead` sub-blocks ahead
//     of the slowest, so the rows the 32 workgroups gather at any time span a few thousand voxels and are fetched into
//     the XCD's L2 once for all offsets.  The wait is bounded: after max_polls polls a workgroup goes on regardless, so
//     the kernel ends whatever the progress words say.  Pacing saves traffic and costs time; max_polls = 0 is the default.
//
// The step sequence of every workgroup is a function of the pair lists alone: fgx_wgrad_sweep_plan builds it once per
// neighbor cache.  Sums are taken in a fixed order (steps in list order, units in ascending order), so results are the
// same on every run; they differ from the block-major kernels' in the order of the fp32 additions.
#include <type_traits>

#include "wgrad_device.h"

namespace fgx {
namespace {

constexpr int kSwStages = 4;         // row ring depth
constexpr int kSwIdxSlots = 8;       // index ring: two slots per loader
constexpr int kSwLoaders = 4;
constexpr int kSwPairs = 64;         // pairs per step
constexpr int kSwStepRing = 256;     // step-list entries held in LDS (four chunks of 64)
constexpr int kSwTurnRows = 16384;   // a workgroup changes units about every so many voxels (a change swaps the accumulators)
constexpr int kSwMaxSlots = 64;      // workgroups per XCD the pacing poll can look at (one lane each)
constexpr int kSwMaxGroups = kXcds * kSwMaxSlots;
constexpr int kSwWaves = 4 + kSwLoaders;     // wavefronts of a sweep workgroup: four multipliers and the loaders
constexpr unsigned kSwSpinMax = 1u << 20;   // looks at a progress word before a wavefront goes on regardless

// Progress words in LDS replace a barrier per step.  Loader w owns ring stage w and counts the steps it has landed
// there (step k is landed[k % S] > k / S); every multiplier counts the steps whose fragments it has read, and a
// loader refills its stage with step k once all four have read step k - S.  A wavefront writes only its own word.
// The LDS executes one wavefront's operations in order and a word is written after the wait for what it announces,
// so whoever sees the count also sees the data.  The roles run up to S - 1 steps apart and nobody waits for a
// wavefront of its own role.
__device__ __forceinline__ void progress_store(uint32_t* word, uint32_t v) {
    const uint32_t addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint32_t*)word;
    asm volatile("ds_write_b32 %0, %1" ::"v"(addr), "v"(v) : "memory");
}
__device__ __forceinline__ uint32_t progress_load(const uint32_t* word) {
    const uint32_t addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint32_t*)word;
    uint32_t w;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(w) : "v"(addr) : "memory");
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)w);
}
__device__ __forceinline__ uint32_t progress_min4(const uint32_t* words) {
    const uint32_t addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint32_t*)words;
    u32x4 w;
    asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(w) : "v"(addr) : "memory");
    const uint32_t a = w[0] < w[1] ? w[0] : w[1], b = w[2] < w[3] ? w[2] : w[3];
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)(a < b ? a : b));
}
// a 32-bit LDS read that is not waited for here: the value may be used after a later wait for LDS reads (they return
// in order) and lds_arrived(), which keeps the compiler from using it earlier
__device__ __forceinline__ uint32_t lds_read_word(const uint32_t* word) {
    const uint32_t addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const uint32_t*)word;
    uint32_t w;
    asm volatile("ds_read_b32 %0, %1" : "=v"(w) : "v"(addr) : "memory");
    return w;
}
__device__ __forceinline__ void lds_arrived(uint32_t& a, uint32_t& b) { asm volatile("" : "+v"(a), "+v"(b)); }
// spins until the minimum of the four words reaches `need`; `known` caches the last minimum seen.  After kSwSpinMax looks
// the wavefront goes on regardless, so that the kernel ends whatever happens, and `gave_up` is set: data it works with from
// then on may be stale, and the reduction turns the whole result into NaN
__device__ __forceinline__ void progress_wait(const uint32_t* words, uint32_t need, uint32_t& known, uint32_t& gave_up) {
    if (known >= need) return;
    for (unsigned spins = 0; spins < kSwSpinMax; ++spins) {
        known = progress_min4(words);
        if (known >= need) return;
        __builtin_amdgcn_s_sleep(1);
    }
    gave_up = 1u;
}

// ------------------------------------------------------------------------------------------------
// Plan: fine bounds, units (parts), per-workgroup step lists
// ------------------------------------------------------------------------------------------------
struct SweepUnit {
    // The 64-pair steps of offset v inside the XCD's voxels are numbered 0, 1, 2, ...; the offset is cut into P slices
    // that take the steps in turn (step j belongs to slice j % P, P <= 64), and a unit owns the slices in `mask`.
    // Units of one offset can so have any sizes, which is what evens out the workgroups' loads.
    uint32_t v, P;
    uint32_t lo, hi;        // pair range of the offset inside the XCD's voxels
    uint32_t nsteps;
    uint32_t mask_lo, mask_hi;
    uint32_t pad;
};
struct SweepGroup {         // one workgroup
    uint32_t step_off, nsteps;
    uint32_t sb0;           // first sub-block of its XCD
    uint32_t active;        // workgroups of its XCD that have steps
};

struct SweepLayout {
    unsigned nsb, groups, spx;
    size_t fine, units, wg, vcount, vlist, steps_k, steps_m, step_cap, total;
};

SweepLayout sweep_layout(size_t n, size_t n_pairs, int V, int sub_rows, int groups) {
    SweepLayout L{};
    L.nsb = n ? cdiv(n, (size_t)sub_rows) : 0u;
    L.groups = (unsigned)groups;
    L.spx = (unsigned)groups / kXcds;
    size_t off = 0;
    L.fine = off;
    off = align_up(off + (size_t)V * (L.nsb + 1) * 4, 256);
    L.units = off;
    off = align_up(off + (size_t)groups * 2 * sizeof(SweepUnit), 256);
    L.wg = off;
    off = align_up(off + (size_t)groups * sizeof(SweepGroup), 256);
    L.vcount = off;
    off = align_up(off + (size_t)kMaxV * 4, 256);
    L.vlist = off;
    off = align_up(off + (size_t)kMaxV * groups * 2 * 2, 256);
    // every unit's steps: at most pairs / 64 whole steps in all plus one ragged step per unit
    L.step_cap = n_pairs / kSwPairs + (size_t)groups * 2 + 64;
    L.steps_k = off;
    off = align_up(off + L.step_cap * 4, 256);
    L.steps_m = off;
    off = align_up(off + L.step_cap * 4, 256);
    L.total = off;
    return L;
}

__device__ __forceinline__ uint64_t unit_mask(const SweepUnit& u) { return ((uint64_t)u.mask_hi << 32) | u.mask_lo; }
// how many of the offset's steps 0 .. J-1 belong to the unit
__device__ __forceinline__ uint32_t unit_count_below(const SweepUnit& u, uint32_t J) {
    if (u.P == 0) return 0;
    const uint32_t full = J / u.P, rem = J % u.P;
    const uint64_t m = unit_mask(u);
    const uint64_t low = rem ? (m & (~0ull >> (64 - rem))) : 0ull;
    return full * (uint32_t)__popcll(m) + (uint32_t)__popcll(low);
}
// the offset-wide number of the unit's t-th step
__device__ __forceinline__ uint32_t unit_step_at(const SweepUnit& u, uint32_t t) {
    uint64_t m = unit_mask(u);
    const uint32_t pc = (uint32_t)__popcll(m);
    const uint32_t cycle = t / pc;
    for (uint32_t r = t % pc; r > 0; --r) m &= m - 1;       // drop the r lowest slices
    return cycle * u.P + (uint32_t)(__ffsll((long long)m) - 1);
}
__device__ __forceinline__ uint32_t offset_steps(uint32_t cnt) { return (cnt + kSwPairs - 1) / kSwPairs; }

// One wavefront per XCD cuts its pair ranges into units, lane v keeping the state of offset v; then the step-list
// offsets and the per-offset lists of partial products are laid out.
constexpr unsigned kSwCumMax = 4096;     // sub-blocks whose running pair counts fit the units kernel's LDS

// k of the slices in `have_mask`, evenly spread over them (all lanes: lane i decides slice i)
__device__ __forceinline__ uint64_t spread_take(uint64_t have_mask, unsigned k, unsigned lane) {
    const unsigned have = (unsigned)__popcll(have_mask);
    if (k >= have) return have_mask;
    const bool mine = (have_mask >> lane) & 1ull;
    const unsigned rank = (unsigned)__popcll(have_mask & ((1ull << lane) - 1ull));      // slices of the mask below this one
    const bool taken = mine && ((rank + 1u) * k / have > rank * k / have);              // where k * rank / have steps up
    return __ballot(taken);
}
// lane holding the smallest (largest) key among the lanes with `live`, lowest lane on ties; -1 if none
__device__ __forceinline__ int wave_arg(bool live, float key, unsigned lane, bool want_max) {
    const uint32_t bits = __builtin_bit_cast(uint32_t, key);                              // keys are >= 0: bits order like values
    unsigned long long k = want_max ? (((unsigned long long)bits << 8) | (255u - lane))
                                    : (((unsigned long long)(~bits) << 8) | (255u - lane));
    if (!live) k = 0ull;
#pragma unroll
    for (int sh = 32; sh > 0; sh >>= 1) {
        const unsigned long long o = __shfl_xor(k, sh, 64);
        k = o > k ? o : k;
    }
    return k == 0ull ? -1 : (int)(255u - (unsigned)(k & 255u));
}

__global__ void __launch_bounds__(64 * kXcds) sweep_units_kernel(const uint32_t* __restrict__ fine, int V, unsigned nsb, unsigned spx,
                                                                SweepUnit* __restrict__ units, SweepGroup* __restrict__ wg,
                                                                uint32_t* __restrict__ vcount, uint16_t* __restrict__ vlist) {
    const unsigned x = threadIdx.x;
    // pairs (all offsets) before every sub-block boundary, by all threads: the XCDs' ranges are cut from it
    __shared__ uint32_t cum[kSwCumMax + 1];
    // what the layout pass below needs of every unit (steps, offset), kept out of global memory
    __shared__ uint32_t sh_steps[kSwMaxGroups * 2];
    __shared__ uint8_t sh_v[kSwMaxGroups * 2];
    const bool by_pairs = nsb <= kSwCumMax;
    if (by_pairs) {
        // (eight offsets' counts fetched together: a loop over a run-time V waits for every load in turn)
        for (unsigned sb = x; sb <= nsb; sb += blockDim.x) {
            uint32_t c = 0;
            for (int v0 = 0; v0 < V; v0 += 8) {
                uint32_t at[8], first[8];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int v = v0 + k < V ? v0 + k : V - 1;
                    at[k] = fine[(size_t)v * (nsb + 1) + sb];
                    first[k] = fine[(size_t)v * (nsb + 1)];
                }
#pragma unroll
                for (int k = 0; k < 8; ++k) c += v0 + k < V ? at[k] - first[k] : 0u;
            }
            cum[sb] = c;
        }
    }
    __syncthreads();
    {
        const unsigned xc = x >> 6, lane = x & 63u;         // wavefront xc plans XCD xc
        // XCD xc takes the sub-blocks [sbA, sbB): boundaries where the running pair count (all offsets) passes xc / 8
        // of the total, so that the XCDs get equal work rather than equal voxel counts
        auto boundary = [&](unsigned q) -> unsigned {
            if (q == 0) return 0u;
            if (q >= (unsigned)kXcds) return nsb;
            if (!by_pairs) return (unsigned)((uint64_t)q * nsb / kXcds);      // (very many sub-blocks: equal voxel counts)
            const uint64_t want = (uint64_t)cum[nsb] * q / kXcds;
            unsigned lo_sb = 0, hi_sb = nsb;            // first sub-block boundary with at least `want` pairs before it
            while (lo_sb < hi_sb) {
                const unsigned mid = (lo_sb + hi_sb) >> 1;
                if (cum[mid] < want) lo_sb = mid + 1;
                else hi_sb = mid;
            }
            return lo_sb;
        };
        const unsigned sbA = boundary(xc), sbB = boundary(xc + 1);
        // Every offset is cut into up to 64 slices that take its steps in turn.  The workgroups are filled one after
        // the other to the average of what is left: the smallest remaining offset whole, topped up with slices of the
        // largest one (or, when the smallest is larger than the average, a share of it alone) -- at most two units per
        // workgroup, loads equal up to a slice.  A workgroup must retire offsets for good when as many remain as the
        // workgroups after it can still take (two each): that keeps the scheme from running out of unit slots.
        uint32_t lo = 0, cnt = 0, N = 0, P = 0;             // this lane's offset
        uint64_t left = 0;                                  // its slices not yet given out
        float per = 0.f;                                    // steps per slice
        if (lane < (unsigned)V) {
            lo = fine[(size_t)lane * (nsb + 1) + sbA];
            cnt = fine[(size_t)lane * (nsb + 1) + sbB] - lo;
            N = offset_steps(cnt);
            P = N < 64u ? N : 64u;
            left = P ? (~0ull >> (64 - P)) : 0ull;
            per = P ? (float)N / (float)P : 0.f;
        }
        float total = (float)N;
#pragma unroll
        for (int sh = 32; sh > 0; sh >>= 1) total += __shfl_xor(total, sh, 64);
        for (unsigned s = 0; s < spx; ++s) {
            const int after = (int)(spx - 1 - s);               // workgroups after this one
            const float want = total / (float)(spx - s);
            const int items = (int)__popcll(__ballot(left != 0));
            const int must_retire = items - 2 * after;
            const float rem = per * (float)__popcll(left);
            const int a = wave_arg(left != 0, rem, lane, false);
            int b = -1;
            uint64_t mask_a = 0, mask_b = 0;
            if (a >= 0) {                                       // (uniform)
                const float rem_a = __shfl(rem, a, 64), per_a = __shfl(per, a, 64);
                const uint64_t left_a = __shfl((unsigned long long)left, a, 64);
                const bool share = rem_a > want && must_retire < 1;     // a share of the smallest offset fills the workgroup
                if (share) {
                    const unsigned k = (unsigned)(want / per_a + 0.5f);
                    mask_a = spread_take(left_a, k ? k : 1u, lane);
                } else {
                    mask_a = left_a;
                }
                if ((int)lane == a) left &= ~mask_a;
                if (!share) {
                    // top up: from the largest other offset, or (when offsets must go) the smallest one whole
                    b = wave_arg(left != 0 && (int)lane != a, rem, lane, must_retire < 2);
                    if (b >= 0) {
                        const float per_b = __shfl(per, b, 64), need = want - rem_a;
                        const uint64_t left_b = __shfl((unsigned long long)left, b, 64);
                        if (must_retire >= 2) mask_b = left_b;
                        else if (need > 0.5f * per_b) mask_b = spread_take(left_b, (unsigned)(need / per_b + 0.5f), lane);
                        if ((int)lane == b) left &= ~mask_b;
                    }
                }
            }
            // lane a writes the first unit, lane b the second (lane 0 an empty one where there is none)
            uint32_t my_steps = 0;
            for (int u = 0; u < 2; ++u) {
                const int who = u == 0 ? a : b;
                const uint64_t mask = u == 0 ? mask_a : mask_b;
                const bool have = who >= 0 && mask != 0;
                if ((int)lane == (have ? who : 0)) {
                    SweepUnit un{};
                    if (have) {
                        un.v = lane;
                        un.P = P;
                        un.lo = lo;
                        un.hi = lo + cnt;
                        un.mask_lo = (uint32_t)mask;
                        un.mask_hi = (uint32_t)(mask >> 32);
                        un.nsteps = unit_count_below(un, N);
                        my_steps += un.nsteps;
                    }
                    const unsigned q = (xc * spx + s) * 2 + (unsigned)u;
                    units[q] = un;
                    sh_steps[q] = un.nsteps;
                    sh_v[q] = (uint8_t)un.v;
                }
            }
            float given = (float)my_steps;
#pragma unroll
            for (int sh = 32; sh > 0; sh >>= 1) given += __shfl_xor(given, sh, 64);
            total -= given;
            if (lane == 0) wg[(size_t)xc * spx + s].sb0 = sbA;
        }
    }
    __syncthreads();
    // step-list offsets: an exclusive running sum over the workgroups' step counts (wavefront 0: 64 lanes x up to 8
    // workgroups each, a shuffle scan across the lanes); active workgroups per XCD: a count per wavefront
    __shared__ uint32_t sh_off[kSwMaxGroups + 1];
    __shared__ uint32_t sh_active[kXcds];
    const unsigned groups = (unsigned)kXcds * spx;
    {
        const unsigned lane = x & 63u;
        if (x < 64u) {
            constexpr unsigned kPer = kSwMaxGroups / 64;
            uint32_t mine[kPer], sum = 0;
#pragma unroll
            for (unsigned k = 0; k < kPer; ++k) {
                const unsigned g = lane * kPer + k;
                mine[k] = g < groups ? sh_steps[g * 2] + sh_steps[g * 2 + 1] : 0u;
                sum += mine[k];
            }
            uint32_t incl = sum;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t up = __shfl_up(incl, d, 64);
                if ((int)lane >= d) incl += up;
            }
            uint32_t off = incl - sum;
#pragma unroll
            for (unsigned k = 0; k < kPer; ++k) {
                const unsigned g = lane * kPer + k;
                if (g < groups) sh_off[g] = off;
                off += mine[k];
            }
        }
        // wavefront xc counts XCD xc's workgroups that have steps (spx <= 64)
        const unsigned xc = x >> 6;
        const bool has = lane < spx && (sh_steps[(xc * spx + lane) * 2] + sh_steps[(xc * spx + lane) * 2 + 1]) != 0u;
        const unsigned long long mask = __ballot(has);
        if (lane == 0) sh_active[xc] = (uint32_t)__popcll(mask);
    }
    __syncthreads();
    for (unsigned g = x; g < groups; g += blockDim.x) {
        wg[g].step_off = sh_off[g];
        wg[g].nsteps = sh_steps[g * 2] + sh_steps[g * 2 + 1];
        wg[g].active = sh_active[g / spx];
    }
    // the partial products of every offset, in ascending unit order (the reduction adds them in this order): a unit's
    // place in its offset's list is the number of units of that offset before it -- counted per wavefront with a ballot
    // per offset, the wavefronts' counts added up in order
    const unsigned total_units = groups * 2;
    __shared__ uint16_t sh_cnt[kMaxV][(kSwMaxGroups * 2) / 64];       // [offset][run of 64 units]
    const unsigned runs = (total_units + 63u) / 64u;
    for (unsigned r0 = 0; r0 < runs; r0 += blockDim.x / 64) {
        const unsigned run = r0 + (x >> 6), q = run * 64 + (x & 63u);
        const bool live = run < runs && q < total_units && sh_steps[q] != 0u;
        const int mine_v = live ? (int)sh_v[q] : -1;
        for (int v = 0; v < V; ++v) {
            const unsigned long long m = __ballot(mine_v == v);
            if ((x & 63u) == 0 && run < runs) sh_cnt[v][run] = (uint16_t)__popcll(m);
        }
    }
    __syncthreads();
    if (x < (unsigned)V) {                 // exclusive sums over the runs, in place; the total is the offset's count
        uint32_t c = 0;
        for (unsigned run = 0; run < runs; ++run) {
            const uint32_t here = sh_cnt[x][run];
            sh_cnt[x][run] = (uint16_t)c;
            c += here;
        }
        vcount[x] = c;
    }
    __syncthreads();
    for (unsigned r0 = 0; r0 < runs; r0 += blockDim.x / 64) {
        const unsigned run = r0 + (x >> 6), q = run * 64 + (x & 63u);
        const bool live = run < runs && q < total_units && sh_steps[q] != 0u;
        const int mine_v = live ? (int)sh_v[q] : -1;
        for (int v = 0; v < V; ++v) {
            const unsigned long long m = __ballot(mine_v == v);
            if (mine_v == v) {
                const unsigned before = (unsigned)__popcll(m & ((1ull << (x & 63u)) - 1ull));
                vlist[(size_t)v * total_units + sh_cnt[v][run] + before] = (uint16_t)q;
            }
        }
    }
}

// number of steps of unit u whose first pair lies below `bound`
__device__ __forceinline__ uint32_t steps_below(const SweepUnit& u, uint32_t bound) {
    if (u.nsteps == 0 || bound <= u.lo) return 0;
    const uint32_t all = offset_steps(u.hi - u.lo);
    uint32_t J = (bound - u.lo + kSwPairs - 1) / kSwPairs;       // steps of the offset that start below the bound
    if (J > all) J = all;
    return unit_count_below(u, J);
}

// The merged step list of one workgroup per block: its two units' steps ordered by the group of sub-blocks their first
// pair lies in, unit 0 first inside a group.  Entry: first pair | pairs in the step (7 bits), unit (1 bit), sub-block relative to
// the XCD's first (24 bits).
__global__ void __launch_bounds__(256) sweep_steps_kernel(const uint32_t* __restrict__ fine, unsigned nsb,
                                                          const SweepUnit* __restrict__ units,
                                                          const SweepGroup* __restrict__ wg, uint32_t* __restrict__ steps_k,
                                                          uint32_t* __restrict__ steps_m, size_t step_cap, unsigned turn_shift) {
    const unsigned g = blockIdx.x;
    const SweepGroup grp = wg[g];
    const SweepUnit u0 = units[(size_t)g * 2], u1 = units[(size_t)g * 2 + 1];
    const unsigned sbA = grp.sb0;
    for (int u = 0; u < 2; ++u) {
        const SweepUnit& me = u == 0 ? u0 : u1;
        const SweepUnit& other = u == 0 ? u1 : u0;
        const uint32_t* mine = fine + (size_t)me.v * (nsb + 1);
        const uint32_t* theirs = fine + (size_t)other.v * (nsb + 1);
        for (uint32_t j = threadIdx.x; j < me.nsteps; j += 256) {
            const uint32_t k = me.lo + unit_step_at(me, j) * kSwPairs;
            const uint32_t left = me.hi - k;
            // sub-block of pair k: the last s with mine[s] <= k (pairs of the XCD start at sub-block sbA)
            unsigned lo = sbA, hi = nsb;            // invariant: mine[lo] <= k, answer in [lo, hi)
            while (hi - lo > 1) {
                const unsigned mid = (lo + hi) >> 1;
                if (mine[mid] <= k) lo = mid;
                else hi = mid;
            }
            const unsigned sb = lo;
            // the two units take turns by groups of 2^turn_shift sub-blocks: the other unit's steps in earlier groups
            // and, for unit 1, in this one (unit 0 goes first)
            const unsigned grp_first = sbA + (((sb - sbA) >> turn_shift) << turn_shift);
            const unsigned grp_end = grp_first + (1u << turn_shift) < nsb ? grp_first + (1u << turn_shift) : nsb;
            const uint32_t before = u == 0 ? steps_below(other, theirs[grp_first]) : steps_below(other, theirs[grp_end]);
            const size_t at = (size_t)grp.step_off + j + before;
            if (at < step_cap) {
                steps_k[at] = k;
                steps_m[at] = (left < (uint32_t)kSwPairs ? left : (uint32_t)kSwPairs) | ((uint32_t)u << 7) | ((sb - sbA) << 8);
            }
        }
    }
}

__global__ void __launch_bounds__(256) sweep_clear_kernel(uint32_t* __restrict__ prog, unsigned n) {
    const unsigned i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) prog[i] = 0u;
}

// ------------------------------------------------------------------------------------------------
// The kernel
// ------------------------------------------------------------------------------------------------
// Exchange two accumulator tiles in place.  Written as register swaps by hand: left to the compiler, "whose sums are
// in the working registers" becomes a copy of a whole tile into a third set of registers before every step and back
// after it.
__device__ __forceinline__ void swap_tiles(f32x16& a, f32x16& b) {
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        float x = a[e], y = b[e];
        asm volatile("v_swap_b32 %0, %1" : "+v"(x), "+v"(y));
        a[e] = x;
        b[e] = y;
    }
#endif
}

// a 16-bit value (the low half of `bits`) as fp32
template <typename Tag> __device__ __forceinline__ float half_to_float(uint32_t bits);
template <> __device__ __forceinline__ float half_to_float<F16>(uint32_t bits) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}
template <> __device__ __forceinline__ float half_to_float<BF16>(uint32_t bits) { return __builtin_bit_cast(float, bits << 16); }
template <> __device__ __forceinline__ float half_to_float<F32>(uint32_t) { return 0.f; }

template <typename Tag, int BM, int BN>
struct SweepCfg {
    using T = typename Tag::type;
    static constexpr int ES = (int)sizeof(T);
    static constexpr int P = kSwPairs, S = kSwStages;
    static constexpr int NW = 4, NL = kSwLoaders, NT = 64 * (NW + NL);
    static constexpr int WM = BM / 2, WN = BN / 2, TM = WM / 32, TN = WN / 32;
    static constexpr int ROWB_A = BM * ES, ROWB_B = BN * ES;
    static constexpr int CH_A = ROWB_A / 16, CH_B = ROWB_B / 16;
    static constexpr int RPI_A = 64 / CH_A, RPI_B = 64 / CH_B;
    static constexpr int A_PER = P / RPI_A / NL, B_PER = P / RPI_B / NL;
    static constexpr int LPS = A_PER + B_PER;
    static constexpr int A_BYTES = P * ROWB_A, B_BYTES = P * ROWB_B, STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int IDX_SLOT_BYTES = 2 * P * 4;               // sig_o x P | sig_i x P
    static constexpr size_t lds_bytes = (size_t)S * STAGE_BYTES + (size_t)kSwIdxSlots * IDX_SLOT_BYTES + (size_t)kSwStepRing * 8 + 32;
    static_assert(NW == 4 && NL == S, "one loader per ring stage; the multipliers' progress words are read four at a time");
    static_assert(ES == 2, "16-bit types");
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert(P % (RPI_A * NL) == 0 && P % (RPI_B * NL) == 0, "every loader issues the same row loads");
    static constexpr int key_a(int row) { return CH_A >= 16 ? 4 * (row & 3) : (CH_A >= 8 ? 2 * (row & 3) : 0); }
    static constexpr int key_b(int row) { return CH_B >= 16 ? 4 * (row & 3) : (CH_B >= 8 ? 2 * (row & 3) : 0); }
};

template <typename Tag, int BM, int BN>
__global__ void __launch_bounds__(64 * (4 + kSwLoaders))
wgrad_sweep_kernel(const typename Tag::type* __restrict__ gout, const typename Tag::type* __restrict__ feats,
                   const uint32_t* __restrict__ sig_i, const uint32_t* __restrict__ sig_o,
                   const SweepUnit* __restrict__ units, const SweepGroup* __restrict__ groups_tab,
                   const uint32_t* __restrict__ steps_k, const uint32_t* __restrict__ steps_m, unsigned spx, int V, int Ci,
                   int Co, uint32_t n_pairs, uint32_t gout_bytes, uint32_t feats_bytes, float* __restrict__ partial,
                   float* __restrict__ bias_partial, int bias_offset, uint32_t* __restrict__ prog, unsigned lead,
                   unsigned max_polls, uint32_t* __restrict__ giveup) {
    using C = SweepCfg<Tag, BM, BN>;
    constexpr int ES = C::ES, S = C::S, P = C::P;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    unsigned char* ring = lds_raw;                                              // [S][A rows | B rows]
    uint32_t* idx_ring = (uint32_t*)(ring + S * C::STAGE_BYTES);                // [kSwIdxSlots][o x P | i x P]
    uint32_t* step_k = idx_ring + kSwIdxSlots * 2 * P;                          // [kSwStepRing] first pair of a step
    uint32_t* step_m = step_k + kSwStepRing;                                    // [kSwStepRing] count | unit | sub-block
    uint32_t* landed = step_m + kSwStepRing;                                    // [NL] steps whose rows have landed, per loader
    uint32_t* consumed = landed + 4;                                            // [NW] steps read, per multiplier

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool loader = wave >= C::NW;
    const int lw = loader ? wave - C::NW : 0, mw = loader ? 0 : wave;
    const int wave_m = mw >> 1, wave_n = mw & 1;
    const int g = lane >> 5, l32 = lane & 31;

    // workgroup ids are dealt round-robin to the XCDs
    const unsigned xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds;
    const unsigned gid = xcd * spx + slot;
    const SweepGroup grp = groups_tab[gid];
    const unsigned nsteps = grp.nsteps;
    uint32_t* my_prog = prog + gid;
    // giveup[workgroup][wavefront]: every wavefront writes its word once, at its end -- 1 if one of its waits for data ran
    // out of looks, else 0 -- so the words need no clearing between calls
    uint32_t* my_giveup = giveup + (size_t)gid * kSwWaves + wave;
    uint32_t gave_up = 0u;
    if (nsteps == 0) {                               // nothing to do: nobody has to wait for this workgroup
        if (tid == 0) __hip_atomic_store(my_prog, 0xFFFFFFFFu, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (lane == 0) *my_giveup = 0u;
        return;
    }

    const rsrc_t gout_rs = make_rsrc(gout, gout_bytes);
    const rsrc_t feats_rs = make_rsrc(feats, feats_bytes);
    const rsrc_t sigo_rs = make_rsrc(sig_o, n_pairs * 4u);
    const rsrc_t sigi_rs = make_rsrc(sig_i, n_pairs * 4u);
    const rsrc_t stepk_rs = make_rsrc(steps_k + grp.step_off, nsteps * 4u);     // reads past the list give zeros
    const rsrc_t stepm_rs = make_rsrc(steps_m + grp.step_off, nsteps * 4u);
    const uint32_t rowb_o = (uint32_t)Co * ES, rowb_i = (uint32_t)Ci * ES;

    // 64 entries of the step list into LDS (chunk c -> ring quarter c & 3)
    auto load_chunk = [&](unsigned c) {
        uint32_t* dk = step_k + (c & 3) * 64;
        uint32_t* dm = step_m + (c & 3) * 64;
        const uint32_t vo = (c * 64 + (uint32_t)lane) * 4u;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(stepk_rs, FGX_LDS_PTR(dk), 4, vo, 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(stepm_rs, FGX_LDS_PTR(dm), 4, vo, 0, 0, 0);
    };

    if (loader) {
        // =============================================================================================
        // loaders
        // =============================================================================================
        if (lw == 0) {
            load_chunk(0);
            load_chunk(1);
            wait_vmcnt<0>();
        } else if (lw == 1 && lane < 8) {
            landed[lane] = 0u;                      // (landed and consumed are adjacent)
        }
        __syncthreads();                            // (1) the first two chunks of the step list are in LDS, progress words zero
        // Loader lw owns ring stage lw and the steps lw, lw + S, lw + 2S, ...: it enqueues all of a step's rows, turns
        // the next step's indices into addresses while they are on their way, and announces the step when they have
        // landed.  The four loaders take turns on the address path, and the per-step scalar work happens once per step
        // and loader, beside the load latency instead of in front of it.
        //
        // Which pair goes to which of a stage's P row slots is free as long as both operands agree (the products are
        // summed over the slots).  Slot i * RPI + sub (load instruction i, row `sub` of its RPI rows) takes pair
        // sub * NA + i of the step: a lane then needs NA consecutive entries of each pair list, which it fetches
        // straight into registers with 16-byte loads, a round ahead -- no index ring in LDS, no LDS round trip.
        constexpr int NA = P / C::RPI_A, NB = P / C::RPI_B;     // load instructions per operand and step
        static_assert(NA == NB && NA % 8 == 0, "one slot order for both operands, indices in 16-byte pieces, column sums eight rows at a time");
        static_assert(NA + NB + NA / 2 + 4 < 64, "outstanding loads exceed the vmcnt range");
        const int sub = lane / C::CH_A;                                    // row inside a load instruction
        // byte column inside the tile, swizzle applied (the key depends on row & 3 alone, an instruction covers 4 or 8 rows)
        const uint32_t a_chb = (uint32_t)(((lane % C::CH_A) ^ C::key_a(sub)) * 16);
        const uint32_t b_chb = (uint32_t)(((lane % C::CH_B) ^ C::key_b(sub)) * 16);
        unsigned char* stage = ring + lw * C::STAGE_BYTES;
        struct Indices {
            u32x4 o[NA / 4], i[NA / 4];
        };
        auto fetch_idx = [&](unsigned k, Indices& ix) {     // this lane's pair-list entries of step k (zeros past the lists)
            const uint32_t first = k < nsteps ? step_k[k & (kSwStepRing - 1)] : n_pairs;
            const uint32_t at = (first + (uint32_t)(sub * NA)) * 4u;
#pragma unroll
            for (int q = 0; q < NA / 4; ++q) {
                ix.o[q] = __builtin_amdgcn_raw_buffer_load_b128(sigo_rs, (int)(at + q * 16u), 0, 0);
                ix.i[q] = __builtin_amdgcn_raw_buffer_load_b128(sigi_rs, (int)(at + q * 16u), 0, 0);
            }
        };
        uint32_t va[NA], vb[NB];
        auto prep_rows = [&](unsigned k, const Indices& ix) {     // buffer offsets of step k's rows (rows and row sizes fit 24 bits)
            if (k >= nsteps) return;
            const uint32_t left = step_m[k & (kSwStepRing - 1)] & 127u;                // pairs in this step
            const bool ragged = left < (uint32_t)P || (uint32_t)(BM * ES) > rowb_o || (uint32_t)(BN * ES) > rowb_i;   // uniform
#pragma unroll
            for (int q = 0; q < NA / 4; ++q) {
                // (whole vectors into scalars first: indexing a vector element inside a cast has been miscompiled)
                const uint32_t o0 = ix.o[q][0], o1 = ix.o[q][1], o2 = ix.o[q][2], o3 = ix.o[q][3];
                const uint32_t i0 = ix.i[q][0], i1 = ix.i[q][1], i2 = ix.i[q][2], i3 = ix.i[q][3];
                va[q * 4 + 0] = __umul24(o0, rowb_o) + a_chb;
                va[q * 4 + 1] = __umul24(o1, rowb_o) + a_chb;
                va[q * 4 + 2] = __umul24(o2, rowb_o) + a_chb;
                va[q * 4 + 3] = __umul24(o3, rowb_o) + a_chb;
                vb[q * 4 + 0] = __umul24(i0, rowb_i) + b_chb;
                vb[q * 4 + 1] = __umul24(i1, rowb_i) + b_chb;
                vb[q * 4 + 2] = __umul24(i2, rowb_i) + b_chb;
                vb[q * 4 + 3] = __umul24(i3, rowb_i) + b_chb;
            }
            if (ragged) {
#pragma unroll
                for (int i = 0; i < NA; ++i) {
                    const bool live = (uint32_t)(sub * NA + i) < left;
                    va[i] = (live && a_chb < rowb_o) ? va[i] : kOobOffset;
                    vb[i] = (live && b_chb < rowb_i) ? vb[i] : kOobOffset;
                }
            }
        };
        auto fire_rows = [&]() {
#pragma unroll
            for (int i = 0; i < NA; ++i) {
                const uint32_t vo = va[i];
                __builtin_amdgcn_raw_ptr_buffer_load_lds(gout_rs, FGX_LDS_PTR(stage + i * 1024), 16, vo, 0, 0, 0);
            }
            unsigned char* stage_b = stage + C::A_BYTES;
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                const uint32_t vo = vb[i];
                __builtin_amdgcn_raw_ptr_buffer_load_lds(feats_rs, FGX_LDS_PTR(stage_b + i * 1024), 16, vo, 0, 0, 0);
            }
        };
        // one round: step k's rows are enqueued, the entries of step k + 2S requested, step k + S prepared from the
        // entries requested a round ago, and step k announced
        // Column sums of grad_out (the bias gradient) ride along with the offset whose pairs hold every output row once.
        // The loaders add them up, not the multipliers: a loader has time to spare between its rounds, a multiplier
        // none (with the sums in the multipliers, the workgroups that held a unit of this offset were the last to
        // finish by a tenth of the kernel).  After announcing a step of that offset the loader reads back what its own
        // loads deposited -- lane l of load instruction i wrote 16 bytes at i * 1024 + 16 * l, the same eight channels
        // for every i -- and adds the NA pairs into eight fp32 sums.  Rows past the end of a step and channels past Co
        // arrived as zeros.  The stage is this loader's own: nobody refills it before its next round.
        const SweepUnit lu0 = units[(size_t)gid * 2], lu1 = units[(size_t)gid * 2 + 1];
        const bool lbias0 = bias_partial != nullptr && lu0.nsteps && (int)lu0.v == bias_offset;
        const bool lbias1 = bias_partial != nullptr && lu1.nsteps && (int)lu1.v == bias_offset;
        float bsum[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) bsum[e] = 0.f;
        auto add_columns = [&]() {
            const unsigned char* mine = stage + lane * 16;
#pragma unroll
            for (int i0 = 0; i0 < NA; i0 += 8) {
                u32x4 piece[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) piece[i] = *(const u32x4*)(mine + (i0 + i) * 1024);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const uint32_t w0 = piece[i][0], w1 = piece[i][1], w2 = piece[i][2], w3 = piece[i][3];
                    bsum[0] += half_to_float<Tag>(w0 & 0xFFFFu);
                    bsum[1] += half_to_float<Tag>(w0 >> 16);
                    bsum[2] += half_to_float<Tag>(w1 & 0xFFFFu);
                    bsum[3] += half_to_float<Tag>(w1 >> 16);
                    bsum[4] += half_to_float<Tag>(w2 & 0xFFFFu);
                    bsum[5] += half_to_float<Tag>(w2 >> 16);
                    bsum[6] += half_to_float<Tag>(w3 & 0xFFFFu);
                    bsum[7] += half_to_float<Tag>(w3 >> 16);
                }
            }
        };
        uint32_t known_consumed = 0;
        auto round = [&](unsigned k, const Indices& ready, Indices& coming) {
            if (k >= (unsigned)S) progress_wait(consumed, k - S + 1u, known_consumed, gave_up);   // every multiplier has read step k - S
            fire_rows();
            // loader 0 also keeps the step list: the chunk after next, whose quarter of the ring was read 128+ steps ago
            if (lw == 0 && (k & 63u) == 0u) load_chunk(k / 64 + 2);
            fetch_idx(k + 2 * S, coming);
            const bool sums = ((step_m[k & (kSwStepRing - 1)] >> 7) & 1u) ? lbias1 : lbias0;       // (uniform)
            prep_rows(k + S, ready);
            wait_vmcnt<0>();
            progress_store(landed + lw, k / S + 1u);
            if (sums) add_columns();
        };

        __syncthreads();                            // (2)
        Indices ix0, ix1;
        fetch_idx((unsigned)lw, ix0);
        fetch_idx((unsigned)lw + S, ix1);
        prep_rows((unsigned)lw, ix0);
        for (unsigned k = (unsigned)lw; k < nsteps; k += 2 * S) {
            round(k, ix1, ix0);
            if (k + S < nsteps) round(k + S, ix0, ix1);
        }
        wait_vmcnt<0>();
        if (lbias0 || lbias1) {
            // bias_partial[workgroup][loader][co].  Row r of a load instruction holds channel piece c in lane
            // r * CH_A + (c ^ key(r)): every lane collects its own piece from all rows, the lanes of row 0 write.
            const int piece = (int)(a_chb >> 4);
            float total[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) total[e] = 0.f;
#pragma unroll
            for (int r = 0; r < C::RPI_A; ++r) {
                const int from = r * C::CH_A + (piece ^ C::key_a(r));
#pragma unroll
                for (int e = 0; e < 8; ++e) total[e] += __shfl(bsum[e], from, 64);
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) bsum[e] = total[e];
            float* bdst = bias_partial + ((size_t)gid * kSwLoaders + lw) * Co;
            const int co0 = (int)(a_chb / ES);
            if (sub == 0) {
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (co0 + e < Co) bdst[co0 + e] = bsum[e];
            }
        }
        if (lane == 0) *my_giveup = gave_up;
        return;
    }

    // =================================================================================================
    // multipliers
    // =================================================================================================
    __syncthreads();                                // (1)
    __syncthreads();                                // (2) the loaders' prologue barriers
    const SweepUnit un0 = units[(size_t)gid * 2], un1 = units[(size_t)gid * 2 + 1];
    const int s16 = lane & 15, mb = (lane >> 4) & 1;
    // Per-lane byte offsets of the transposing reads inside a stage, for k-block 0 and the first of a lane's two pair
    // rows; the second pair row (4 rows on: same swizzle key) and the k-block go into the instruction's offset field.
    uint32_t a_off[C::TM], b_off[C::TN];
    {
        const int prow = g * 8 + (s16 >> 2);
        static_assert(C::key_a(0) == C::key_a(4) && C::key_b(1) == C::key_b(5), "pair rows 4 apart share a swizzle key");
#pragma unroll
        for (int i = 0; i < C::TM; ++i) {
            const int byte = (wave_m * C::WM + i * 32 + mb * 16 + (s16 & 3) * 4) * 2;
            const int c = byte >> 4, w = byte & 15;
            a_off[i] = (uint32_t)(prow * C::ROWB_A + ((c ^ C::key_a(prow)) << 4) + w);
        }
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
            const int byte = (wave_n * C::WN + j * 32 + mb * 16 + (s16 & 3) * 4) * 2;
            const int c = byte >> 4, w = byte & 15;
            b_off[j] = (uint32_t)(C::A_BYTES + prow * C::ROWB_B + ((c ^ C::key_b(prow)) << 4) + w);
        }
    }
    constexpr int NK = P / 16;                      // k-blocks (16 pair rows) per step
    constexpr int RK = 2 * (C::TM + C::TN);         // LDS reads per k-block

    // `acc` is the accumulator of the unit whose steps are being multiplied, `rest` that of the other one: the two
    // change places when the step list changes units (a handful of times per sub-block), so that the multiply code
    // exists once and the register allocator sees one set of MFMA destinations.
    f32x16 acc[C::TM][C::TN], rest[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i) {
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                acc[i][j][e] = 0.f;
                rest[i][j][e] = 0.f;
            }
    }
    unsigned acc_unit = 0;                          // whose sums `acc` holds

    // Fragments of one k-block (16 pair rows): TM x 2 reads of the grad_out tile, TN x 2 of the feats tile.
    i16x4 fr[2][RK];
    // (the k-block is a compile-time constant: it is part of the instructions' offset fields)
    auto read_block = [&](const uint32_t stage_addr, auto kk_c, i16x4 (&dst)[RK]) {
        constexpr int kk = decltype(kk_c)::value;
#pragma unroll
        for (int i = 0; i < C::TM; ++i) {
            dst[i * 2] = lds_read_tr16_at<kk * 16 * C::ROWB_A>(stage_addr + a_off[i]);
            dst[i * 2 + 1] = lds_read_tr16_at<kk * 16 * C::ROWB_A + 4 * C::ROWB_A>(stage_addr + a_off[i]);
        }
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
            dst[(C::TM + j) * 2] = lds_read_tr16_at<kk * 16 * C::ROWB_B>(stage_addr + b_off[j]);
            dst[(C::TM + j) * 2 + 1] = lds_read_tr16_at<kk * 16 * C::ROWB_B + 4 * C::ROWB_B>(stage_addr + b_off[j]);
        }
    };
    using K0 = std::integral_constant<int, 0>;
    using K1 = std::integral_constant<int, 1>;
    using K2 = std::integral_constant<int, 2>;
    using K3 = std::integral_constant<int, 3>;
    const uint32_t ring_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const unsigned char*)ring;
    // the products of one k-block
    auto multiply_block = [&](i16x4 (&f)[RK]) {
#pragma unroll
        for (int i = 0; i < C::TM; ++i) {
            const i16x8 af = __builtin_shufflevector(f[i * 2], f[i * 2 + 1], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
            for (int j = 0; j < C::TN; ++j) {
                const i16x8 bf = __builtin_shufflevector(f[(C::TM + j) * 2], f[(C::TM + j) * 2 + 1], 0, 1, 2, 3, 4, 5, 6, 7);
                mma16<Tag>(acc[i][j], af, bf);
            }
        }
    };

    // pacing state of the first multiplier (values in `prog`: sub-block + 1; 0 = not started, all ones = finished)
    uint32_t cur_sb = step_m[0] >> 8, known_min = 0;
    bool pacing = mw == 0 && max_polls > 0 && grp.active > 1;
    if (mw == 0 && lane == 0) __hip_atomic_store(my_prog, cur_sb + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t* xcd_prog = prog + xcd * spx;

    auto run_steps = [&]() {
        static_assert(NK == 4, "the step below is written out for four k-blocks");
        // The fragment reads run one k-block ahead of the products and do not stop at the end of a step: while the last
        // k-block of a step is multiplied the first one of the next step arrives.
        uint32_t meta = step_m[0];
        {
            unsigned spins = 0;
            for (; spins < kSwSpinMax && progress_load(landed) < 1u; ++spins) __builtin_amdgcn_s_sleep(1);
            if (spins == kSwSpinMax) gave_up = 1u;      // went on without the first step's rows
        }
        read_block(ring_addr, K0{}, fr[0]);
        lds_wait_but<0>(fr[0]);
        for (unsigned step = 0; step < nsteps; ++step) {
            const uint32_t cur = ring_addr + (step & (S - 1)) * (uint32_t)C::STAGE_BYTES;
            const uint32_t nxt = ring_addr + ((step + 1) & (S - 1)) * (uint32_t)C::STAGE_BYTES;
            const bool more = step + 1 < nsteps;
            const unsigned unit = (meta >> 7) & 1u;
            if (unit != acc_unit) {
                acc_unit = unit;
                // (the swaps are assembly the compiler does not see into: let the last products leave the pipe first)
#pragma unroll
                for (int q = 0; q < 3; ++q) asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
                for (int i = 0; i < C::TM; ++i)
#pragma unroll
                    for (int j = 0; j < C::TN; ++j) swap_tiles(acc[i][j], rest[i][j]);
            }
            read_block(cur, K1{}, fr[1]);
            multiply_block(fr[0]);       // (landed before the loop came round)
            // the next step's list entry and its stage's progress word travel with the fragments of the third k-block
            uint32_t next_meta = lds_read_word(step_m + ((step + 1) & (kSwStepRing - 1)));
            uint32_t seen = lds_read_word(landed + ((step + 1) & (S - 1)));
            read_block(cur, K2{}, fr[0]);
            lds_wait_but<RK>(fr[1]);
            lds_arrived(next_meta, seen);
            multiply_block(fr[1]);
            read_block(cur, K3{}, fr[1]);
            lds_wait_but<RK>(fr[0]);
            multiply_block(fr[0]);
            if (more && (uint32_t)__builtin_amdgcn_readfirstlane((int)seen) < (step + 1) / S + 1u) {     // the loaders are behind: wait here
                unsigned spins = 0;
                for (; spins < kSwSpinMax && progress_load(landed + ((step + 1) & (S - 1))) < (step + 1) / S + 1u; ++spins)
                    __builtin_amdgcn_s_sleep(1);
                if (spins == kSwSpinMax) gave_up = 1u;      // goes on with whatever the stage holds
            }
            read_block(nxt, K0{}, fr[0]);                      // (after the last step: read and never used)
            lds_wait_but<RK>(fr[1]);
            progress_store(consumed + mw, step + 1u);       // the stage has been read: its loader may refill it
            multiply_block(fr[1]);
            // The prefetched fragments land while these products run.  They are waited for before the loop goes round:
            // registers with a read in flight must not cross the loop edge, where the compiler may copy them.
            lds_wait_but<0>(fr[0]);
            meta = (uint32_t)__builtin_amdgcn_readfirstlane((int)next_meta);
            next_meta = meta;
            // Pacing, by the first multiplier before its next step (while it waits its progress word stands still, the
            // loaders run out of free stages after S - 1 steps and the other multipliers out of landed ones, so the
            // whole workgroup is held back with it): tell the XCD which sub-block this workgroup is entering, and do
            // not enter one more than `lead` ahead of the slowest workgroup.  Bounded: after max_polls looks the
            // workgroup stops pacing.
            if (mw == 0 && step + 1 < nsteps) {
                const uint32_t next_sb = next_meta >> 8;
                if (next_sb != cur_sb) {
                    cur_sb = next_sb;
                    if (lane == 0) __hip_atomic_store(my_prog, cur_sb + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (pacing && cur_sb > known_min + lead) {
                        unsigned polls = 0;
                        while (true) {
                            uint32_t seen = 0xFFFFFFFFu;
                            if ((unsigned)lane < spx) seen = __hip_atomic_load(xcd_prog + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
                            for (int sh = 32; sh > 0; sh >>= 1) {
                                const uint32_t o = (uint32_t)__shfl_xor((int)seen, sh, 64);
                                seen = o < seen ? o : seen;
                            }
                            known_min = seen ? seen - 1u : 0u;
                            if (cur_sb <= known_min + lead) break;
                            if (++polls >= max_polls) {
                                pacing = false;         // give up for good: the kernel must end whatever the others do
                                break;
                            }
                            __builtin_amdgcn_s_sleep(32);
                        }
                    }
                }
            }
        }
    };
    run_steps();
    if (mw == 0 && lane == 0) __hip_atomic_store(my_prog, 0xFFFFFFFFu, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // partial[unit][co][ci], fp32
    auto store_acc = [&](f32x16 (&a)[C::TM][C::TN], unsigned q) {
        float* dst = partial + (size_t)q * ((size_t)Co * Ci);
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
            const int ci = wave_n * C::WN + j * 32 + l32;
            if (ci >= Ci) continue;
#pragma unroll
            for (int i = 0; i < C::TM; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int co = wave_m * C::WM + i * 32 + (e >> 2) * 8 + g * 4 + (e & 3);
                    if (co < Co) dst[(size_t)co * Ci + ci] = a[i][j][e];
                }
        }
    };
    if (acc_unit == 0) {
        if (un0.nsteps) store_acc(acc, gid * 2);
        if (un1.nsteps) store_acc(rest, gid * 2 + 1);
    } else {
        if (un0.nsteps) store_acc(rest, gid * 2);
        if (un1.nsteps) store_acc(acc, gid * 2 + 1);
    }
    if (lane == 0) *my_giveup = gave_up;
}

// grad_weight[co][v][ci] = sum of the partial products of offset v's units, in a fixed order.  Four lanes per four
// adjacent ci, four loads in flight each.  The blocks from `weight_blocks` on (present when a bias gradient is asked
// for) take one column of grad_bias each: the sum over the workgroups that held a unit of the bias offset (four
// loaders' sums each), two workgroups per thread, then a tree over LDS -- a fixed order of additions.
// Every block first looks at the sweep's give-up words (one per wavefront): if any is set, a wavefront went on without the
// data it waited for, and every weight and bias gradient is written as NaN instead of a sum that may be wrong.
template <typename T>
__global__ void __launch_bounds__(256) sweep_reduce_kernel(const float* __restrict__ partial,
                                                           const uint32_t* __restrict__ vcount,
                                                           const uint16_t* __restrict__ vlist, unsigned total_units, int V,
                                                           int Ci, int Co, T* __restrict__ gw, unsigned weight_blocks,
                                                           const float* __restrict__ bias_partial,
                                                           const SweepUnit* __restrict__ units, unsigned groups,
                                                           int bias_offset, T* __restrict__ gbias,
                                                           const uint32_t* __restrict__ giveup) {
    static_assert(kSwMaxGroups == 512 && kSwLoaders == 4, "two workgroups per thread, four sums per workgroup");
    uint32_t flags = 0u;
    for (unsigned i = threadIdx.x; i < groups * kSwWaves; i += 256) flags |= giveup[i];
    const bool poisoned = __syncthreads_or(flags != 0u) != 0;
    const float poison = __builtin_nanf("");
    if (blockIdx.x >= weight_blocks) {
        __shared__ float sums[256];
        const int co = (int)(blockIdx.x - weight_blocks);
        float pair[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const unsigned gidx = threadIdx.x + h * 256;
            pair[h] = 0.f;
            if (gidx < groups) {
                const SweepUnit a = units[(size_t)gidx * 2], b = units[(size_t)gidx * 2 + 1];
                const bool has = (a.nsteps && (int)a.v == bias_offset) || (b.nsteps && (int)b.v == bias_offset);
                if (has) {
                    const float* p = bias_partial + (size_t)gidx * kSwLoaders * Co + co;        // one sum per loader
                    pair[h] = (p[0] + p[Co]) + (p[2 * (size_t)Co] + p[3 * (size_t)Co]);
                }
            }
        }
        sums[threadIdx.x] = pair[0] + pair[1];
        __syncthreads();
        for (unsigned half = 128; half > 0; half >>= 1) {
            if (threadIdx.x < half) sums[threadIdx.x] += sums[threadIdx.x + half];
            __syncthreads();
        }
        if (threadIdx.x == 0) gbias[co] = from_float<T>(poisoned ? poison : sums[0]);
        return;
    }
    const size_t quads = (size_t)Co * V * (Ci / 4);
    const size_t per = (size_t)Co * Ci;
    // four adjacent lanes share a quad: lane j adds the units j, j + 4, ... of the list, the four sums are then added as
    // (0 + 1) + (2 + 3)
    const unsigned part = threadIdx.x & 3u;
    for (size_t t = ((size_t)blockIdx.x * 256 + threadIdx.x) >> 2; t < quads; t += (size_t)weight_blocks * 64) {
        const int cq = (int)(t % (Ci / 4));
        const size_t r = t / (Ci / 4);
        const int v = (int)(r % V), co = (int)(r / V);
        const unsigned cnt = vcount[v];
        const uint16_t* list = vlist + (size_t)v * total_units;
        const float* src = partial + (size_t)co * Ci + cq * 4;
        float4 s = {0.f, 0.f, 0.f, 0.f};
        unsigned i = part;
        for (; i + 12 < cnt; i += 16) {
            float4 x[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) x[q] = *(const float4*)(src + (size_t)list[i + 4 * q] * per);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                s.x += x[q].x;
                s.y += x[q].y;
                s.z += x[q].z;
                s.w += x[q].w;
            }
        }
        for (; i < cnt; i += 4) {
            const float4 x = *(const float4*)(src + (size_t)list[i] * per);
            s.x += x.x;
            s.y += x.y;
            s.z += x.z;
            s.w += x.w;
        }
#pragma unroll
        for (int sh = 1; sh <= 2; sh <<= 1) {
            s.x += __shfl_xor(s.x, sh, 64);
            s.y += __shfl_xor(s.y, sh, 64);
            s.z += __shfl_xor(s.z, sh, 64);
            s.w += __shfl_xor(s.w, sh, 64);
        }
        if (poisoned) s.x = s.y = s.z = s.w = poison;
        if (part == 0) {
            T* dst = gw + ((size_t)co * V + v) * Ci + cq * 4;
            dst[0] = from_float<T>(s.x);
            dst[1] = from_float<T>(s.y);
            dst[2] = from_float<T>(s.z);
            dst[3] = from_float<T>(s.w);
        }
    }
}

struct SweepScratch {
    size_t prog, giveup, partial, bias, colsum, total;
};
SweepScratch sweep_scratch(int Ci, int Co, int groups) {
    SweepScratch S{};
    size_t off = 0;
    S.prog = off;
    off = align_up(off + (size_t)groups * 4, 256);
    S.giveup = off;
    off = align_up(off + (size_t)groups * kSwWaves * 4, 256);
    S.partial = off;
    off = align_up(off + (size_t)groups * 2 * Co * Ci * sizeof(float), 256);
    S.bias = off;
    off = align_up(off + (size_t)groups * kSwLoaders * Co * sizeof(float), 256);
    S.colsum = off;
    off += fgx_colsum_scratch_bytes(0, Co);
    S.total = off;
    return S;
}

int sweep_groups() {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    int g = cus / kXcds * kXcds;
    if (g > kSwMaxGroups) g = kSwMaxGroups;
    return g;
}

bool tile_ok(int tile, int Ci, int Co) { return (tile == 128 || tile == 64) && Ci <= tile && Co <= tile; }

// the second half of a sweep: the units' partial products (and the loaders' column sums, if `gbias`) in `scratch` -> gradients
template <typename T>
int launch_sweep_reduce(const char* plan, const SweepLayout& L, int V, int Ci, int Co, char* scratch, const SweepScratch& S,
                        void* gw, void* gbias, int bias_offset, hipStream_t s) {
    const float* partial = (const float*)(scratch + S.partial);
    const float* bias_partial = gbias ? (const float*)(scratch + S.bias) : nullptr;
    const size_t quads = (size_t)Co * V * (Ci / 4);
    unsigned grid = cdiv(quads * 4, 256);      // four lanes per quad of weights
    sweep_reduce_kernel<T><<<grid + (bias_partial ? (unsigned)Co : 0u), 256, 0, s>>>(
        partial, (const uint32_t*)(plan + L.vcount), (const uint16_t*)(plan + L.vlist), L.groups * 2, V, Ci, Co, (T*)gw, grid,
        bias_partial, (const SweepUnit*)(plan + L.units), L.groups, bias_offset, (T*)gbias,
        (const uint32_t*)(scratch + S.giveup));
    FGX_CHECK_LAUNCH("fgx_conv_wgrad_sweep(reduce)");
    return FGX_OK;
}

template <typename Tag, int BM, int BN>
int launch_sweep(const void* gout, const void* feats, const uint32_t* sig_i, const uint32_t* sig_o, const char* plan,
                 const SweepLayout& L, size_t n, size_t n_in, uint32_t n_pairs, int V, int Ci, int Co, char* scratch,
                 const SweepScratch& S, void* gw, void* gbias, int bias_offset, int lead, int max_polls, hipStream_t s) {
    using C = SweepCfg<Tag, BM, BN>;
    using T = typename Tag::type;
    auto kern = wgrad_sweep_kernel<Tag, BM, BN>;
    static thread_local bool lds_raised = false;
    if (C::lds_bytes > 64 * 1024 && !lds_raised) {
        FGX_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)C::lds_bytes));
        lds_raised = true;
    }
    uint32_t* prog = (uint32_t*)(scratch + S.prog);
    float* partial = (float*)(scratch + S.partial);
    float* bias_partial = gbias ? (float*)(scratch + S.bias) : nullptr;
    const SweepUnit* units = (const SweepUnit*)(plan + L.units);
    if (max_polls > 0) {       // the pacing words; nobody looks at them otherwise
        sweep_clear_kernel<<<cdiv(L.groups, 256), 256, 0, s>>>(prog, L.groups);
        FGX_CHECK_LAUNCH("fgx_conv_wgrad_sweep(clear)");
    }
    kern<<<L.groups, C::NT, C::lds_bytes, s>>>((const T*)gout, (const T*)feats, sig_i, sig_o, units,
                                               (const SweepGroup*)(plan + L.wg), (const uint32_t*)(plan + L.steps_k),
                                               (const uint32_t*)(plan + L.steps_m), L.spx, V, Ci, Co, n_pairs,
                                               (uint32_t)(n * (size_t)Co * sizeof(T)), (uint32_t)(n_in * (size_t)Ci * sizeof(T)),
                                               partial, bias_partial, bias_offset, prog, (unsigned)lead, (unsigned)max_polls,
                                               (uint32_t*)(scratch + S.giveup));
    FGX_CHECK_LAUNCH("fgx_conv_wgrad_sweep");
    return launch_sweep_reduce<T>(plan, L, V, Ci, Co, scratch, S, gw, gbias, bias_offset, s);
}

}  // namespace
}  // namespace fgx

using namespace fgx;

extern "C" {

size_t fgx_wgrad_sweep_plan_bytes(size_t n, size_t n_pairs, int V, int sub_rows) {
    const int groups = sweep_groups();
    if (V < 1 || V > kMaxV || sub_rows < 1 || groups < kXcds) return 0;
    return sweep_layout(n, n_pairs, V, sub_rows, groups).total;
}

int fgx_wgrad_sweep_plan(const uint32_t* sig_o, const uint32_t* seg_host, size_t n, int V, int sub_rows, void* plan,
                         size_t plan_bytes, fgx_stream_t stream) {
    FGX_CHECK_ARG(V >= 1 && V <= kMaxV, "fgx_wgrad_sweep_plan: bad kernel volume %d", V);
    FGX_CHECK_ARG(sub_rows >= 64, "fgx_wgrad_sweep_plan: sub_rows must be at least 64, got %d", sub_rows);
    FGX_CHECK_ARG(seg_host && plan, "fgx_wgrad_sweep_plan: null buffer");
    FGX_CHECK_ARG(n > 0 && n < 0xFFFFFFFFull, "fgx_wgrad_sweep_plan: row count out of range");
    FGX_CHECK_ARG(((uintptr_t)plan & 255) == 0, "fgx_wgrad_sweep_plan: plan must be 256-byte aligned");
    SegTable tab;
    for (int v = 0; v <= V; ++v) {
        FGX_CHECK_ARG(v == 0 || seg_host[v] >= seg_host[v - 1], "fgx_wgrad_sweep_plan: segment table is not monotone");
        tab.seg[v] = seg_host[v];
    }
    for (int v = V + 1; v <= kMaxV; ++v) tab.seg[v] = seg_host[V];
    const size_t n_pairs = seg_host[V];
    FGX_CHECK_ARG(n_pairs == seg_host[0] || sig_o != nullptr, "fgx_wgrad_sweep_plan: null pair list");
    FGX_CHECK_ARG(seg_host[0] == 0, "fgx_wgrad_sweep_plan: the segment table must start at 0");
    const int groups = sweep_groups();
    FGX_CHECK_ARG(groups >= kXcds && groups / kXcds * 2 >= V, "fgx_wgrad_sweep_plan: too few compute units for %d offsets", V);
    const SweepLayout L = sweep_layout(n, n_pairs, V, sub_rows, groups);
    FGX_CHECK_ARG((size_t)L.nsb + 1 < (1u << 24), "fgx_wgrad_sweep_plan: too many sub-blocks; use larger sub_rows");
    FGX_CHECK_ARG(plan_bytes >= L.total, "fgx_wgrad_sweep_plan: plan of %zu bytes, need %zu", plan_bytes, L.total);
    hipStream_t s = (hipStream_t)stream;
    char* p = (char*)plan;
    uint32_t* fine = (uint32_t*)(p + L.fine);
    PhaseEnd phases{s};
    phase_mark("wgrad sweep plan", s);
    block_bounds_kernel<<<cdiv((size_t)V * (L.nsb + 1), 256), 256, 0, s>>>(sig_o, tab, V, L.nsb, (unsigned)sub_rows, fine);
    FGX_CHECK_LAUNCH("fgx_wgrad_sweep_plan(bounds)");
    sweep_units_kernel<<<1, 64 * kXcds, 0, s>>>(fine, V, L.nsb, L.spx, (SweepUnit*)(p + L.units), (SweepGroup*)(p + L.wg),
                                        (uint32_t*)(p + L.vcount), (uint16_t*)(p + L.vlist));
    FGX_CHECK_LAUNCH("fgx_wgrad_sweep_plan(units)");
    unsigned turn_shift = 0;
    while (turn_shift < 16 && ((size_t)sub_rows << turn_shift) < (size_t)kSwTurnRows) ++turn_shift;
    sweep_steps_kernel<<<L.groups, 256, 0, s>>>(fine, L.nsb, (const SweepUnit*)(p + L.units), (const SweepGroup*)(p + L.wg),
                                                (uint32_t*)(p + L.steps_k), (uint32_t*)(p + L.steps_m), L.step_cap, turn_shift);
    FGX_CHECK_LAUNCH("fgx_wgrad_sweep_plan(steps)");
    return FGX_OK;
}

size_t fgx_wgrad_sweep_scratch_bytes(int Ci, int Co) {
    const int groups = sweep_groups();
    if (Ci <= 0 || Co <= 0 || groups < kXcds) return 0;
    return sweep_scratch(Ci, Co, groups).total;
}

int fgx_conv_wgrad_sweep(int dtype, const void* grad_out, const void* feats, const uint32_t* sig_i, const uint32_t* sig_o,
                         const uint32_t* seg_host, const void* plan, size_t n, size_t n_in, int Ci, int Co, int V, int tile,
                         int sub_rows, int lead, int max_polls, void* scratch, void* grad_weight, void* grad_bias,
                         int bias_offset, fgx_stream_t stream) {
    FGX_CHECK_ARG(dtype == FGX_F16 || dtype == FGX_BF16, "fgx_conv_wgrad_sweep: 16-bit types only (dtype %d)", dtype);
    FGX_CHECK_ARG(Ci > 0 && Co > 0 && V >= 1 && V <= kMaxV, "fgx_conv_wgrad_sweep: bad shape Ci=%d Co=%d V=%d", Ci, Co, V);
    FGX_CHECK_ARG(tile_ok(tile, Ci, Co), "fgx_conv_wgrad_sweep: a single %dx%d tile does not hold Co=%d x Ci=%d", tile, tile, Co, Ci);
    FGX_CHECK_ARG(Ci % 8 == 0 && Co % 8 == 0, "fgx_conv_wgrad_sweep: rows of %d / %d elements are not multiples of 16 bytes", Ci, Co);
    FGX_CHECK_ARG(sub_rows >= 64 && lead >= 0 && max_polls >= 0, "fgx_conv_wgrad_sweep: bad pacing arguments");
    FGX_CHECK_ARG(seg_host && plan && scratch && grad_weight, "fgx_conv_wgrad_sweep: null buffer");
    // (the loaders multiply row numbers with 24-bit multiplies)
    FGX_CHECK_ARG(n > 0 && n <= (1ull << 24) && n_in <= (1ull << 24), "fgx_conv_wgrad_sweep: at most 2^24 rows per operand (n=%zu, n_in=%zu)", n, n_in);
    FGX_CHECK_ARG(((uintptr_t)scratch & 255) == 0 && ((uintptr_t)plan & 255) == 0, "fgx_conv_wgrad_sweep: scratch and plan must be 256-byte aligned");
    const size_t n_pairs = seg_host[V];
    FGX_CHECK_ARG(n_pairs > 0 && grad_out && feats && sig_i && sig_o, "fgx_conv_wgrad_sweep: empty pair lists or null buffer");
    FGX_CHECK_ARG((((uintptr_t)grad_out | (uintptr_t)feats) & 15) == 0, "fgx_conv_wgrad_sweep: grad_out and feats must be 16-byte aligned");
    FGX_CHECK_ARG((double)n * Co * 2 <= (double)kOobOffset && (double)n_in * Ci * 2 <= (double)kOobOffset &&
                      (double)n_pairs * 4 + 256 <= (double)kOobOffset,
                  "fgx_conv_wgrad_sweep: an operand exceeds the 32-bit offset range; use fgx_conv_wgrad");
    const int groups = sweep_groups();
    FGX_CHECK_ARG(groups >= kXcds && groups / kXcds * 2 >= V, "fgx_conv_wgrad_sweep: too few compute units for %d offsets", V);
    const SweepLayout L = sweep_layout(n, n_pairs, V, sub_rows, groups);
    const SweepScratch S = sweep_scratch(Ci, Co, groups);
    hipStream_t s = (hipStream_t)stream;
    void* fused_bias = nullptr;
    if (grad_bias != nullptr) {
        const bool fuse = bias_offset >= 0 && bias_offset < V && (size_t)(seg_host[bias_offset + 1] - seg_host[bias_offset]) == n;
        if (fuse) fused_bias = grad_bias;
        else {
            int rc = fgx_colsum(dtype, grad_out, n, Co, (char*)scratch + S.colsum, grad_bias, stream);
            if (rc != FGX_OK) return rc;
        }
    }
#define FGX_SWEEP(TAG, T_)                                                                                                      \
    if (tile == T_)                                                                                                             \
        return launch_sweep<TAG, T_, T_>(grad_out, feats, sig_i, sig_o, (const char*)plan, L, n, n_in, (uint32_t)n_pairs, V, Ci, Co, \
                                         (char*)scratch, S, grad_weight, fused_bias, bias_offset, lead, max_polls, s);
    if (dtype == FGX_F16) { FGX_SWEEP(F16, 128) FGX_SWEEP(F16, 64) }
    else { FGX_SWEEP(BF16, 128) FGX_SWEEP(BF16, 64) }
#undef FGX_SWEEP
    set_error("fgx_conv_wgrad_sweep: no kernel for tile %d", tile);
    return FGX_ERR_UNSUPPORTED;
}

size_t fgx_wgrad_sweep_giveup_words(int Ci, int Co, size_t* byte_offset) {
    const int groups = sweep_groups();
    if (Ci <= 0 || Co <= 0 || groups < kXcds) return 0;
    if (byte_offset) *byte_offset = sweep_scratch(Ci, Co, groups).giveup;
    return (size_t)groups * kSwWaves;
}

int fgx_wgrad_sweep_reduce(int dtype, const void* plan, size_t n, size_t n_pairs, int Ci, int Co, int V, int sub_rows,
                           void* scratch, void* grad_weight, void* grad_bias, int bias_offset, fgx_stream_t stream) {
    FGX_CHECK_ARG(dtype == FGX_F16 || dtype == FGX_BF16, "fgx_wgrad_sweep_reduce: 16-bit types only (dtype %d)", dtype);
    FGX_CHECK_ARG(Ci > 0 && Co > 0 && Ci % 8 == 0 && Co % 8 == 0 && V >= 1 && V <= kMaxV, "fgx_wgrad_sweep_reduce: bad shape Ci=%d Co=%d V=%d", Ci, Co, V);
    FGX_CHECK_ARG(sub_rows >= 64 && n > 0 && n_pairs > 0, "fgx_wgrad_sweep_reduce: bad sizes");
    FGX_CHECK_ARG(plan && scratch && grad_weight, "fgx_wgrad_sweep_reduce: null buffer");
    FGX_CHECK_ARG(((uintptr_t)scratch & 255) == 0 && ((uintptr_t)plan & 255) == 0, "fgx_wgrad_sweep_reduce: scratch and plan must be 256-byte aligned");
    const int groups = sweep_groups();
    FGX_CHECK_ARG(groups >= kXcds && groups / kXcds * 2 >= V, "fgx_wgrad_sweep_reduce: too few compute units for %d offsets", V);
    const SweepLayout L = sweep_layout(n, n_pairs, V, sub_rows, groups);
    const SweepScratch S = sweep_scratch(Ci, Co, groups);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FGX_F16)
        return launch_sweep_reduce<F16::type>((const char*)plan, L, V, Ci, Co, (char*)scratch, S, grad_weight, grad_bias, bias_offset, s);
    return launch_sweep_reduce<BF16::type>((const char*)plan, L, V, Ci, Co, (char*)scratch, S, grad_weight, grad_bias, bias_offset, s);
}

}  // extern "C"
