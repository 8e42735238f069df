// Streaming masked implicit GEMM (forward and dgrad) for large voxel counts on gfx950.
//
//   out[order[r], :] = sum over offsets v present for row r of src[map[order[r], v], :] x panel_v (+ bias)
//
// Same arithmetic as the tiled kernel in conv_gemm.hip, organised for one resident workgroup per CU:
//
//  * A workgroup is persistent.  It walks its share of the (row tile, column tile) items -- item g, g + G, ... for
//    workgroup g of G -- and treats all their (offset, K-slab) steps as ONE stream: the loads of the next item's first
//    steps are in flight while the last steps of the current item are multiplied and its output tile is written, so
//    neither the start-up latency of a tile nor its epilogue leaves the memory pipeline empty.
//  * The wavefronts are specialised.  WAVES_M x WAVES_N of them only multiply (LDS fragment reads + MFMA) and write
//    the output tiles; kLoaders more (one per SIMD) only enqueue loads.  Issuing a vector-memory instruction blocks
//    its wavefront while the address pipeline is busy, and the loads of a step keep that pipeline busy for about as
//    long as its MFMAs take -- in separate wavefronts the two run side by side instead of one after the other.
//  * The per-tile neighbor indices come from the gather plan (fgx_gather_plan_fill): for every tile and every offset
//    present in it, the tile's source rows as one contiguous run.  An index column is therefore one small contiguous
//    load, fetched kPlanAhead offsets ahead of the rows that need it.
//  * Every load is a buffer load that writes straight into LDS (lane i deposits 16 bytes at LDS base + 16 * i).  A
//    missing neighbor is an out-of-range buffer offset, which the hardware answers with zeros; the per-lane address
//    of a row is a 32-bit offset computed once per offset and reused for all its K-slabs through the scalar offset
//    operand, and the weight-panel and index loads use lane-constant offsets.
//  * No load returns into a register, so a loader's vector-memory counter sees only its own loads in issue order:
//    "the rows of step c have landed" is s_waitcnt vmcnt(number of loads this wavefront issued in the last
//    iteration), chosen among a few immediates by a scalar branch, followed by one workgroup barrier per step.
//
// Stage layout, swizzle, MFMA fragment mapping and the epilogue through LDS are those of the tiled kernel.  The
// output tile is staged in the ring stage that was multiplied last (free until the next enqueue targets it).
#include "gemm_device.h"

namespace fgx {
namespace {

constexpr int kPlanSlots = 4;        // index ring depth
constexpr int kPlanAhead = 3;        // the index stream runs this many offsets ahead of the row stream
constexpr uint32_t kOobOffset = 0xFF000000u;   // buffer offset no source tensor reaches: the load returns zeros
constexpr int kBandSlots = 8;        // band-mask ring depth: a mask is read up to (stages - 2) steps after it was written
constexpr int kStreamStages = 3;     // ring stages (for the short-row tiles 4, 5 and 7 measured the same)
constexpr int kLoaders = 4;          // loader wavefronts per workgroup (one per SIMD)

using rsrc_t = __amdgpu_buffer_rsrc_t;

__device__ __forceinline__ rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), (short)0, (int)bytes, 0x00020000);
}

// multiplier wavefronts along the rows of the 256 x 128 tile with 128-byte slabs: 4 (x 2 along the columns: eight
// multipliers with 64 x 64 wave tiles), or 2 (four multipliers with 128 x 64 wave tiles: 6 instead of 8 fragment reads
// per 8 products)
#ifndef FGX_BIG_WAVES_M
#define FGX_BIG_WAVES_M 4
#endif

template <typename Tag, int BM, int BN, int WAVES_M, int WAVES_N, int CH>
struct StreamCfg {
    using T = typename Tag::type;
    static constexpr int S = kStreamStages;
    static constexpr int ES = (int)sizeof(T);
    static constexpr int NW = WAVES_M * WAVES_N;               // multiplying wavefronts
    static constexpr int NL = kLoaders;
    static constexpr int NT = 64 * (NW + NL);
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int TM = WM / 32, TN = WN / 32;
    static constexpr int SLAB = CH * 16;
    static constexpr int SK = SLAB / ES;
    static constexpr int ROWS_PER_INST = 64 / CH;
    static constexpr int A_PER = BM / ROWS_PER_INST / NL;
    static constexpr int B_INST = BN / ROWS_PER_INST;          // wave-wide loads per panel slab, dealt round-robin to the loaders
    static constexpr int B_PER = (B_INST + NL - 1) / NL;       // ... so a loader issues B_PER of them, or one fewer
    static constexpr int LPS = A_PER + B_PER;                  // most row loads per loader and step
    static constexpr int IDX_INST = BM / 64;                   // wave-wide dword loads per index column
    static constexpr int OROW_INST = (WM + 63) / 64;           // wave-wide dword loads for a wave tile's output rows
    static constexpr int STAGE_BYTES = (BM + BN) * SLAB;
    static constexpr int IDX_SLOT_BYTES = BM * 4;
    static constexpr int OUT_PITCH = WN * ES + 16;
    // rows staged per epilogue pass: the most of 32, 16, 8 whose bands (one per multiplier) fit one ring stage
    static constexpr int BAND_ROWS = NW * 32 * OUT_PITCH <= (BM + BN) * SLAB ? 32 : (NW * 16 * OUT_PITCH <= (BM + BN) * SLAB ? 16 : 8);
    static constexpr int OUT_BAND_BYTES = BAND_ROWS * OUT_PITCH;
    static constexpr int OROW_BYTES = 2 * NW * OROW_INST * 256;
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert(BM % (ROWS_PER_INST * NL) == 0 && BN % ROWS_PER_INST == 0, "rows and panel columns must be whole wave-wide loads");
    static_assert(BM % 64 == 0 && IDX_INST <= NL, "index column must be whole wave-wide loads, one per loader");
    static_assert(NW * OUT_BAND_BYTES <= STAGE_BYTES, "the output bands must fit one ring stage");
    static_assert(LPS + 1 < 64, "vmcnt is a 6-bit counter");
    static_assert(CH == 4 || CH == 8, "slab must be 64 or 128 bytes");
    // (the loaders' wait -- "all but the last iteration's loads have landed" -- is what fixes S at 3 or more)
    static_assert(S >= 3 && S - 1 < kBandSlots, "a band mask must outlive the S - 2 steps between its writing and its reading");
    static constexpr size_t fixed_lds = (size_t)S * STAGE_BYTES + (size_t)kPlanSlots * IDX_SLOT_BYTES + OROW_BYTES + kBandSlots * 4;
};

// s_waitcnt vmcnt(n) for a wave-uniform n in [LO, HI]: the count is an immediate, so a binary tree of scalar branches
// picks the instruction.
template <int LO, int HI>
__device__ __forceinline__ void wait_vmcnt_in(int n) {
    if constexpr (LO == HI) {
        wait_vmcnt<LO>();
    } else {
        constexpr int MID = (LO + HI) / 2;
        if (n <= MID) wait_vmcnt_in<LO, MID>(n);
        else wait_vmcnt_in<MID + 1, HI>(n);
    }
}

__device__ __forceinline__ void wg_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <typename Tag, int BM, int BN, int WAVES_M, int WAVES_N, int CH>
__global__ void __launch_bounds__(64 * (WAVES_M * WAVES_N + kLoaders))
gather_gemm_stream_kernel(const typename Tag::type* __restrict__ src, const typename Tag::type* __restrict__ panel,
                          const typename Tag::type* __restrict__ bias, const int64_t* __restrict__ order,
                          const int32_t* __restrict__ plan_seg, const int32_t* __restrict__ tile_code,
                          const uint32_t* __restrict__ plan_idx, const uint32_t* __restrict__ plan_band, uint32_t n, int K,
                          int cols, int cols_pad,
                          unsigned row_tiles, unsigned col_tiles, uint32_t src_bytes, uint32_t panel_bytes,
                          uint32_t plan_bytes, const uint32_t* __restrict__ item_at, int act,
                          typename Tag::type* __restrict__ out, uint8_t* __restrict__ relu_mask) {
    using C = StreamCfg<Tag, BM, BN, WAVES_M, WAVES_N, CH>;
    using T = typename Tag::type;
    constexpr int S = C::S, kSlabBytes = C::SLAB, kChunks = CH;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    unsigned char* ring = lds_raw;                                          // [S][A: BM x SLAB | B: BN x SLAB]
    uint32_t* idx_ring = (uint32_t*)(ring + S * C::STAGE_BYTES);            // [kPlanSlots][BM] source rows of one offset
    uint32_t* orow_lds = idx_ring + kPlanSlots * BM;                        // [2][NW][OROW_INST * 64] output rows
    uint32_t* band_lds = orow_lds + C::OROW_BYTES / 4;                      // [kBandSlots] band masks, loaders -> multipliers
    float* bias_lds = (float*)(band_lds + kBandSlots);                      // [cols_pad]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool loader = wave >= C::NW;                          // wave-uniform role
    const int lw = loader ? wave - C::NW : 0;                   // loader number
    const int mw = loader ? 0 : wave;                           // multiplier number
    const int wave_m = mw / WAVES_N, wave_n = mw % WAVES_N;
    const int g = lane >> 5, l32 = lane & 31;

    const unsigned total_items = row_tiles * col_tiles;
    const unsigned G = gridDim.x;
    const int slabs = (K + C::SK - 1) / C::SK;
    const uint32_t row_bytes = (uint32_t)K * sizeof(T);
    const bool ragged = (row_bytes % kSlabBytes) != 0;
    if (blockIdx.x >= total_items) return;                      // whole workgroup
    // Workgroups are dealt round-robin to the 8 XCDs.  Give the workgroups of one XCD neighboring items in every
    // round (first items (g % 8) * G/8 + g / 8), so that tiles which gather from the same region share an L2.
    const unsigned first_item = G % kXcds == 0 ? (blockIdx.x % kXcds) * (G / kXcds) + blockIdx.x / kXcds : blockIdx.x;
    // A workgroup takes the positions first_item, first_item + G, ... of the item sequence.  Which (row tile, column
    // tile) sits at a position is the caller's choice (item_at: a permutation of the items, made so that the workgroups'
    // loads come out even); without one, items are walked from the LAST tile down: in the mask-sorted order the late
    // tiles carry the most offsets, so the incomplete final round is made of the cheapest tiles.
    auto locate = [&](unsigned position, unsigned& t, unsigned& ct) {
        const unsigned item = item_at != nullptr ? item_at[position] : total_items - 1 - position;
        t = item / col_tiles;
        ct = item - t * col_tiles;
    };

    const rsrc_t src_rs = make_rsrc(src, src_bytes);
    const rsrc_t panel_rs = make_rsrc(panel, panel_bytes);
    const rsrc_t plan_rs = make_rsrc(plan_idx, plan_bytes);
    const rsrc_t order_rs = make_rsrc(order, n * 8u);

    for (int c = tid; c < cols_pad; c += C::NT) bias_lds[c] = (bias != nullptr && c < cols) ? to_float<T>(bias[c]) : 0.f;

    // =================================================================================================
    // Loader state (meaningful in loader wavefronts only)
    // =================================================================================================
    const int sub_row = lane / kChunks, pch = lane % kChunks;
    int a_row[C::A_PER];
    uint32_t a_choff[C::A_PER], a_voff[C::A_PER], b_voff[C::B_PER];
#pragma unroll
    for (int i = 0; i < C::A_PER; ++i) {
        a_row[i] = (i * C::NL + lw) * C::ROWS_PER_INST + sub_row;
        a_choff[i] = (uint32_t)((pch ^ swz_key<CH>(a_row[i])) << 4);
        a_voff[i] = kOobOffset;
    }
#pragma unroll
    for (int i = 0; i < C::B_PER; ++i) {
        const int col = (i * C::NL + lw) * C::ROWS_PER_INST + sub_row;
        b_voff[i] = (uint32_t)(col * kSlabBytes + ((pch ^ swz_key<CH>(col)) << 4));
    }
    const uint32_t idx_voff = (uint32_t)((lw * 64 + lane) * 4);             // used by loaders < IDX_INST only
    const bool idx_wave = loader && lw < C::IDX_INST;

    // ---- the index stream: walks the plan rows of this workgroup's items, kPlanAhead offsets ahead of the rows ----
    // The offsets of a tile are the set bits of its code (a tile without any owns one all-missing plan row, walked as
    // offset 0), so one scalar load per item feeds the whole walk.
    unsigned f_it = first_item, f_t, f_ct;
    locate(f_it, f_t, f_ct);
    bool f_live = true;
    int f_pos = plan_seg[f_t], f_ring = 0;
    uint32_t f_code = (uint32_t)tile_code[f_t];
    f_code = f_code ? f_code : 1u;
    // queue of offsets the row stream has not started yet (head first)
    int q_v[kPlanAhead], q_ct[kPlanAhead];
    uint32_t q_band[kPlanAhead];
    bool q_live[kPlanAhead];
    auto fetch_slot = [&](int& v, int& ct, uint32_t& band, bool& live) -> int {     // returns the loads this wavefront issued
        live = f_live;
        v = 0;
        ct = 0;
        band = 0;
        if (!f_live) return 0;
        band = plan_band != nullptr ? plan_band[f_pos] : 0xFFFFFFFFu;
        v = __builtin_ctz(f_code);
        f_code &= f_code - 1;
        ct = (int)f_ct;
        int ops = 0;
        if (idx_wave) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(plan_rs, FGX_LDS_PTR(idx_ring + f_ring * BM + lw * 64), 4, idx_voff,
                                                     (uint32_t)f_pos * (uint32_t)(BM * 4), 0, 0);
            ops = 1;
        }
        f_ring = (f_ring + 1) & (kPlanSlots - 1);
        ++f_pos;
        if (f_code == 0) {
            f_it += G;
            f_live = f_it < total_items;
            if (f_live) {
                locate(f_it, f_t, f_ct);
                f_pos = plan_seg[f_t];
                f_code = (uint32_t)tile_code[f_t];
                f_code = f_code ? f_code : 1u;
            }
        }
        return ops;
    };

    // ---- the row stream: S-1 steps ahead of the multiply stream ----
    // slot_begin() makes the next offset current (per-lane row offsets from its index column, panel offset) and
    // starts the index load of the offset kPlanAhead further on; issue_step() enqueues the loads of the current step
    // and moves on by one K-slab.
    bool p_ready = false;
    int p_slab = 0, p_ring = 0, p_band = 0, p_stage = 0;
    uint32_t a_soff = 0, b_soff = 0, cur_band = 0;
    const uint32_t b_slab_stride = (uint32_t)cols_pad * kSlabBytes;
    auto slot_begin = [&]() -> int {
        p_ready = q_live[0];
        if (!p_ready) return 0;
        const int v = q_v[0], ct = q_ct[0];
        cur_band = q_band[0];
#pragma unroll
        for (int i = 0; i + 1 < kPlanAhead; ++i) {
            q_v[i] = q_v[i + 1];
            q_ct[i] = q_ct[i + 1];
            q_band[i] = q_band[i + 1];
            q_live[i] = q_live[i + 1];
        }
        const uint32_t* slot = idx_ring + p_ring * BM;
        // for the multipliers, who fetch it at least two barriers from now; the reads of the index column below are
        // waited for before this wavefront reaches its next barrier, and LDS finishes a wavefront's accesses in order
        if (lw == 0 && lane == 0) band_lds[p_band] = cur_band;
        p_band = (p_band + 1) & (kBandSlots - 1);
        p_ring = (p_ring + 1) & (kPlanSlots - 1);
#pragma unroll
        for (int i = 0; i < C::A_PER; ++i) {
            const uint32_t m = slot[a_row[i]];
            a_voff[i] = m == FGX_EMPTY32 ? kOobOffset : m * row_bytes + a_choff[i];
        }
        p_slab = 0;
        a_soff = 0;
        // wave-uniform by construction; saying so keeps the panel loads from being wrapped in per-lane loops
        b_soff = __builtin_amdgcn_readfirstlane(((uint32_t)(v * slabs) * (uint32_t)cols_pad + (uint32_t)(ct * BN)) * kSlabBytes);
        return fetch_slot(q_v[kPlanAhead - 1], q_ct[kPlanAhead - 1], q_band[kPlanAhead - 1], q_live[kPlanAhead - 1]);
    };
    auto issue_step = [&]() -> int {                     // returns the loads this wavefront issued
        if (!p_ready) return 0;
        unsigned char* stage = ring + p_stage * C::STAGE_BYTES;
        const bool tail = ragged && p_slab == slabs - 1;     // wave-uniform
        int ops = 0;
#pragma unroll
        for (int i = 0; i < C::A_PER; ++i) {
            // 32-row band of this load's rows (a constant when the loaders' loads of one round make up one band)
            const int band = C::NL * C::ROWS_PER_INST == 32 ? i : ((i * C::NL + lw) * C::ROWS_PER_INST) >> 5;
            // the multipliers skip a band none of whose rows has the offset, so the loaders skip it too: nothing to load,
            // and the stage keeps stale data nobody reads
            if (!((cur_band >> band) & 1u)) continue;
            uint32_t vo = a_voff[i];
            if (tail) vo = a_soff + a_choff[i] < row_bytes ? vo : kOobOffset;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(src_rs, FGX_LDS_PTR(stage + (i * C::NL + lw) * 1024), 16, vo, a_soff, 0, 0);
            ++ops;
        }
        unsigned char* stage_b = stage + BM * kSlabBytes;
#pragma unroll
        for (int i = 0; i < C::B_PER; ++i) {
            if (C::B_INST % C::NL != 0 && i * C::NL + lw >= C::B_INST) continue;     // narrow panels: not every loader has one
            const uint32_t vo = b_voff[i];
            __builtin_amdgcn_raw_ptr_buffer_load_lds(panel_rs, FGX_LDS_PTR(stage_b + (i * C::NL + lw) * 1024), 16, vo, b_soff, 0, 0);
            ++ops;
        }
        a_soff += kSlabBytes;
        b_soff = __builtin_amdgcn_readfirstlane(b_soff + b_slab_stride);
        p_stage = p_stage + 1 == S ? 0 : p_stage + 1;
        if (++p_slab == slabs) ops += slot_begin();
        return ops;
    };
    // at most `n` of this loader's loads may still be outstanding; n is wave-uniform, 0 .. LPS + 1
    auto wait_loads = [&](int n) { wait_vmcnt_in<0, C::LPS + 1>(n); };

    // =================================================================================================
    // Multiplier state
    // =================================================================================================
    // output rows of an item's wave tile: one (or two) small loads into this wavefront's own LDS area
    auto fetch_orow = [&](unsigned t, int parity) {
#pragma unroll
        for (int j = 0; j < C::OROW_INST; ++j) {
            const int r = j * 64 + lane;
            const uint32_t row = t * (uint32_t)BM + (uint32_t)(wave_m * C::WM + r);
            const uint32_t vo = (r < C::WM && row < n) ? row * 8u : kOobOffset;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(order_rs, FGX_LDS_PTR(orow_lds + ((parity * C::NW + mw) * C::OROW_INST + j) * 64),
                                                     4, vo, 0, 0, 0);
        }
    };
    int a_frag[kChunks / 2][C::TM], b_frag[kChunks / 2][C::TN];   // byte offsets of this lane's fragments in a stage
#pragma unroll
    for (int kk = 0; kk < kChunks / 2; ++kk) {
#pragma unroll
        for (int i = 0; i < C::TM; ++i) a_frag[kk][i] = swz<CH>(wave_m * C::WM + i * 32 + l32, kk * 2 + g);
#pragma unroll
        for (int j = 0; j < C::TN; ++j) b_frag[kk][j] = BM * kSlabBytes + swz<CH>(wave_n * C::WN + j * 32 + l32, kk * 2 + g);
    }
    constexpr int PIECES = C::WN * C::ES / 16;                // 16-byte pieces per band row
    constexpr int ROWS_PER_PASS = 64 / PIECES;
    const bool vec_ok = (cols * C::ES) % 16 == 0;             // output rows start on 16-byte boundaries

    // ---- item walk.  Both roles walk the same items and meet at the same barriers in the same order, but each runs
    // its own loop, so that neither role's registers stay live through the other's code. ----
    struct Item {
        unsigned it, t, ct;
        int slots;
    };
    Item cur_item{first_item, 0, 0, 0};
    locate(cur_item.it, cur_item.t, cur_item.ct);
    cur_item.slots = __popc((uint32_t)tile_code[cur_item.t]);
    auto following = [&](const Item& c, Item& nx) -> bool {     // the item G positions further on; false past the end
        nx.it = c.it + G;
        nx.t = nx.ct = 0;
        nx.slots = 0;
        if (nx.it >= total_items) return false;
        locate(nx.it, nx.t, nx.ct);
        nx.slots = __popc((uint32_t)tile_code[nx.t]);
        return true;
    };

    if (loader) {
        // the loaders are the critical path and issue few instructions: let them win the issue arbitration against the
        // two multiplier wavefronts of their SIMD (measured: 1 % to 4 % per launch)
        __builtin_amdgcn_s_setprio(3);
        // ---- prologue: index columns of the first kPlanAhead offsets, then the rows of the first S-1 steps ----
#pragma unroll
        for (int i = 0; i < kPlanAhead; ++i) (void)fetch_slot(q_v[i], q_ct[i], q_band[i], q_live[i]);
        wait_vmcnt<0>();
        __syncthreads();          // index columns landed; also publishes bias_lds
        (void)slot_begin();
        int ops_prev = 0;
#pragma unroll
        for (int s = 0; s < S - 1; ++s) {
            wait_vmcnt<0>();
            __syncthreads();
            ops_prev = issue_step();
        }
        while (true) {
            const int nsteps = (cur_item.slots > 0 ? cur_item.slots : 1) * slabs;
            Item nx;
            const bool has_next = following(cur_item, nx);
            for (int s = 0; s < nsteps; ++s) {
                // everything this loader issued before its previous iteration has landed: its share of this step's rows
                wait_loads(ops_prev);
                wg_barrier();              // ... and everybody else's; the stage multiplied in the previous step is free
                ops_prev = issue_step();
            }
            wg_barrier();                  // the multipliers' "done reading the last stage"
            if (!has_next) break;
            cur_item = nx;
        }
        wait_vmcnt<0>();
        return;
    }

    // ---- multipliers ----
    fetch_orow(cur_item.t, 0);
    wait_vmcnt<0>();
    __syncthreads();
#pragma unroll
    for (int s = 0; s < S - 1; ++s) __syncthreads();

    int cur_stage = 0, parity = 0;
    // position in the band-mask ring, K-slab inside the current offset, this wavefront's bits of the offset's mask
    constexpr uint32_t kMineAll = (1u << C::TM) - 1u;
    int m_ring = 1, m_slab = 0;
    uint32_t m_mine = kMineAll, m_next = band_lds[0];
    while (true) {
        const int nsteps = (cur_item.slots > 0 ? cur_item.slots : 1) * slabs;
        // the item after this one (its output rows are fetched now, its size is read now)
        Item nx;
        const bool has_next = following(cur_item, nx);
        const unsigned c_t = cur_item.t, c_ct = cur_item.ct, n_t = nx.t;
        f32x16 acc[C::TM][C::TN];
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
            for (int j = 0; j < C::TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
        if (has_next) fetch_orow(n_t, parity ^ 1);
        for (int s = 0; s < nsteps; ++s) {
            wg_barrier();              // the loaders saw this step's rows land
            const unsigned char* cur = ring + cur_stage * C::STAGE_BYTES;
            cur_stage = cur_stage + 1 == S ? 0 : cur_stage + 1;
            if (m_slab == 0) m_mine = (__builtin_amdgcn_readfirstlane(m_next) >> (wave_m * C::TM)) & kMineAll;
            m_slab = m_slab + 1 == slabs ? 0 : m_slab + 1;
            // last K-slab of an offset: fetch the mask of the next one (published at least two barriers ago); the
            // wait for this step's fragments covers it
            if (m_slab == 0) {
                m_next = band_lds[m_ring];
                m_ring = (m_ring + 1) & (kBandSlots - 1);
            }
            if (m_mine != 0) {
                // band by band: a 32-row band of the wave tile none of whose rows has the offset is neither read nor
                // multiplied (for a given accumulator the products still come in the order of the K-blocks)
                u32x4 af[kChunks / 2][C::TM], bf[kChunks / 2][C::TN];
#pragma unroll
                for (int kk = 0; kk < kChunks / 2; ++kk)
#pragma unroll
                    for (int j = 0; j < C::TN; ++j) bf[kk][j] = *(const u32x4*)(cur + b_frag[kk][j]);
#pragma unroll
                for (int i = 0; i < C::TM; ++i) {
                    if (C::TM > 1 && !((m_mine >> i) & 1u)) continue;
#pragma unroll
                    for (int kk = 0; kk < kChunks / 2; ++kk) af[kk][i] = *(const u32x4*)(cur + a_frag[kk][i]);
                }
#pragma unroll
                for (int i = 0; i < C::TM; ++i) {
                    if (C::TM > 1 && !((m_mine >> i) & 1u)) continue;
#pragma unroll
                    for (int kk = 0; kk < kChunks / 2; ++kk)
#pragma unroll
                        for (int j = 0; j < C::TN; ++j) mma<Tag>(acc[i][j], bf[kk][j], af[kk][i]);   // transposed tile
                }
            }
        }

        // ---- epilogue.  The MFMAs ran with the operands swapped, so a 32x32 accumulator holds the TRANSPOSED
        // tile: element e of lane l belongs to output row l%32 and column 8*(e/4) + 4*(l/32) + e%4 -- four
        // adjacent columns per (lane, e/4), which go to LDS as one 8- or 16-byte store.
        wait_vmcnt<0>();               // this item's output rows (fetched an item ago) and older stores
        wg_barrier();                  // everybody is done reading the last stage
        const int last = cur_stage == 0 ? S - 1 : cur_stage - 1;
        unsigned char* band = ring + last * C::STAGE_BYTES + mw * C::OUT_BAND_BYTES;
        const uint32_t* my_orow = orow_lds + (parity * C::NW + mw) * C::OROW_INST * 64;
        const int col0 = (int)c_ct * BN + wave_n * C::WN;
        constexpr int HALVES = 32 / C::BAND_ROWS;
#pragma unroll
        for (int ih = 0; ih < C::TM * HALVES; ++ih) {
            const int i = ih / HALVES, h = ih % HALVES;      // 32-row tile, half of it
            if (HALVES == 1 || l32 / C::BAND_ROWS == h) {
                const int r = l32 - h * C::BAND_ROWS;
#pragma unroll
                for (int j = 0; j < C::TN; ++j)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int c = j * 32 + q * 8 + g * 4;                   // first of four columns
                        const f32x4 bv = *(const f32x4*)(bias_lds + col0 + c);
                        T pk[4];
                        pk[0] = from_float<T>(activate(acc[i][j][q * 4 + 0] + bv.x, act));
                        pk[1] = from_float<T>(activate(acc[i][j][q * 4 + 1] + bv.y, act));
                        pk[2] = from_float<T>(activate(acc[i][j][q * 4 + 2] + bv.z, act));
                        pk[3] = from_float<T>(activate(acc[i][j][q * 4 + 3] + bv.w, act));
                        unsigned char* dstp = band + r * C::OUT_PITCH + c * C::ES;
                        if constexpr (C::ES == 2) *(uint64_t*)dstp = __builtin_bit_cast(uint64_t, pk);
                        else *(u32x4*)dstp = __builtin_bit_cast(u32x4, pk);
                    }
            }
            // same wavefront wrote and reads: program order inside the wavefront suffices for LDS
#pragma unroll
            for (int pass = 0; pass < C::BAND_ROWS / ROWS_PER_PASS; ++pass) {
                const int r = pass * ROWS_PER_PASS + lane / PIECES;
                const int piece = lane % PIECES;
                const int tr = i * 32 + h * C::BAND_ROWS + r;                      // row inside the wave tile
                const bool live = c_t * (uint32_t)BM + (uint32_t)(wave_m * C::WM + tr) < n;
                const uint32_t orow = my_orow[tr];
                const int col = col0 + piece * (16 / C::ES);
                if (!live || col >= cols) continue;
                const unsigned char* sp = band + r * C::OUT_PITCH + piece * 16;
                T* dp = out + (size_t)orow * cols + col;
                if (vec_ok && col + 16 / C::ES <= cols) {
                    // (streaming store: the output is not read again by this launch and should not push source rows out of L2)
                    const u32x4 piece16 = *(const u32x4*)sp;
                    __builtin_nontemporal_store(piece16, (u32x4*)dp);
                    // one bit per output for the activation's derivative (16-bit types, whole pieces only: the host
                    // passes a mask for such shapes alone)
                    if (C::ES == 2 && relu_mask != nullptr)
                        relu_mask[((size_t)orow * cols + col) >> 3] = (uint8_t)positive_bits16<PositiveLimit<T>::value>(piece16);
                } else {
                    for (int t = 0; t < 16 / C::ES && col + t < cols; ++t) dp[t] = ((const T*)sp)[t];
                }
            }
        }
        if (!has_next) break;
        cur_item = nx;
        parity ^= 1;
    }
    wait_vmcnt<0>();
}

// As many workgroups as the CUs hold at once (the narrow tiles leave room for two per CU: their steps are short, and a
// second stream fills the time the first spends at its barriers).
template <typename Tag, int BM, int BN, int WAVES_M, int WAVES_N, int CH>
int resident_groups(size_t lds, int* groups) {
    using C = StreamCfg<Tag, BM, BN, WAVES_M, WAVES_N, CH>;
    auto kern = gather_gemm_stream_kernel<Tag, BM, BN, WAVES_M, WAVES_N, CH>;
    static thread_local int per_cu = 0;          // per thread and instantiation, for the LDS size it was asked with
    static thread_local size_t per_cu_lds = 0;
    int dev = 0, cus = 0;
    FGX_CHECK_HIP(hipGetDevice(&dev));
    FGX_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    if (per_cu == 0 || per_cu_lds != lds) {
        if (lds > 64 * 1024) FGX_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        int q = 1;
        FGX_CHECK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&q, (const void*)kern, C::NT, lds));
        per_cu = q < 1 ? 1 : (q > 2 ? 2 : q);
        per_cu_lds = lds;
    }
    *groups = (cus > 0 ? cus : 256) * per_cu;
    return FGX_OK;
}

template <typename Tag, int BM, int BN, int WAVES_M, int WAVES_N, int CH>
int launch_stream(const void* src, const void* panel, const void* bias, const int64_t* order, const int32_t* plan_seg,
                  const int32_t* tile_code, const uint32_t* plan_idx, const uint32_t* plan_band, size_t plan_rows, size_t n,
                  size_t n_src, int K, int cols, int cols_pad, size_t panel_bytes, const uint32_t* item_at, int max_groups,
                  int act, void* out, uint8_t* relu_mask, hipStream_t s) {
    using C = StreamCfg<Tag, BM, BN, WAVES_M, WAVES_N, CH>;
    using T = typename Tag::type;
    auto kern = gather_gemm_stream_kernel<Tag, BM, BN, WAVES_M, WAVES_N, CH>;
    const size_t lds = C::fixed_lds + (size_t)cols_pad * sizeof(float);
    if (lds > 160 * 1024) {
        set_error("fgx_conv_gather_gemm_stream: %d output columns need %zu bytes of LDS (limit 163840)", cols, lds);
        return FGX_ERR_UNSUPPORTED;
    }
    static thread_local size_t lds_raised = 0;   // raise the dynamic LDS limit once per thread, instantiation and size
    if (lds > 64 * 1024 && lds > lds_raised) {
        FGX_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        lds_raised = lds;
    }
    const unsigned row_tiles = cdiv(n, BM), col_tiles = cdiv(cols, BN);
    const size_t total = (size_t)row_tiles * col_tiles;
    if (max_groups <= 0) {
        int rc = resident_groups<Tag, BM, BN, WAVES_M, WAVES_N, CH>(lds, &max_groups);
        if (rc != FGX_OK) return rc;
    }
    unsigned groups = (unsigned)(total < (size_t)max_groups ? total : (size_t)max_groups);
    kern<<<groups, C::NT, lds, s>>>((const T*)src, (const T*)panel, (const T*)bias, order, plan_seg, tile_code, plan_idx,
                                    plan_band, (uint32_t)n, K, cols, cols_pad, row_tiles, col_tiles,
                                    (uint32_t)(n_src * (size_t)K * sizeof(T)), (uint32_t)panel_bytes,
                                    (uint32_t)(plan_rows * BM * 4), item_at, act, (T*)out, relu_mask);
    FGX_CHECK_LAUNCH("fgx_conv_gather_gemm_stream");
    return FGX_OK;
}

template <typename Tag>
int dispatch_stream(int tile_rows, int tile_cols, int slab_bytes, const void* src, const void* panel, const void* bias,
                    const int64_t* order, const int32_t* plan_seg, const int32_t* tile_code, const uint32_t* plan_idx,
                    const uint32_t* plan_band, size_t plan_rows, size_t n, size_t n_src, int K, int cols, int cols_pad,
                    size_t panel_bytes, const uint32_t* item_at, int max_groups, int act, void* out, uint8_t* relu_mask,
                    hipStream_t s) {
#define FGX_STREAM_TILE(BM, BN, WMv, WNv, CHv)                                                                          \
    if (tile_rows == BM && tile_cols == BN && slab_bytes == CHv * 16)                                                   \
        return launch_stream<Tag, BM, BN, WMv, WNv, CHv>(src, panel, bias, order, plan_seg, tile_code, plan_idx, plan_band,  \
                                                         plan_rows, n, n_src, K, cols, cols_pad, panel_bytes, item_at, max_groups, act, out, relu_mask, s);
    FGX_STREAM_TILE(256, 128, FGX_BIG_WAVES_M, 2, 8)
    FGX_STREAM_TILE(256, 64, 4, 2, 8)
    FGX_STREAM_TILE(128, 256, 2, 4, 8)      // few voxels, wide outputs: half the rows per tile pad less
    FGX_STREAM_TILE(256, 128, 4, 2, 4)      // 64-byte K-slabs: rows shorter than 128 bytes
    FGX_STREAM_TILE(256, 64, 4, 2, 4)
    FGX_STREAM_TILE(256, 32, 8, 1, 4)
#undef FGX_STREAM_TILE
    set_error("fgx_conv_gather_gemm_stream: no kernel for tile %dx%d with %d-byte slabs", tile_rows, tile_cols, slab_bytes);
    return FGX_ERR_UNSUPPORTED;
}

}  // namespace
}  // namespace fgx

using namespace fgx;

extern "C" int fgx_conv_gather_gemm_stream(int dtype, const void* src, const void* panel, const void* bias,
                                           const int64_t* order, const int32_t* tile_code, const int32_t* plan_seg,
                                           const uint32_t* plan_idx, const uint32_t* plan_band, size_t plan_rows, size_t n,
                                           size_t n_src, int K, int cols, int V,
                                           int tile_rows, int tile_cols, int slab_bytes, const uint32_t* item_at,
                                           int max_groups, void* out, fgx_stream_t stream) {
    return fgx_conv_gather_gemm_stream_act(dtype, src, panel, bias, order, tile_code, plan_seg, plan_idx, plan_band, plan_rows,
                                           n, n_src, K, cols, V, tile_rows, tile_cols, slab_bytes, item_at, max_groups,
                                           FGX_ACT_NONE, out, stream);
}

extern "C" int fgx_conv_gather_gemm_stream_act(int dtype, const void* src, const void* panel, const void* bias,
                                               const int64_t* order, const int32_t* tile_code, const int32_t* plan_seg,
                                               const uint32_t* plan_idx, const uint32_t* plan_band, size_t plan_rows,
                                               size_t n, size_t n_src, int K, int cols, int V,
                                               int tile_rows, int tile_cols, int slab_bytes, const uint32_t* item_at,
                                               int max_groups, int activation, void* out, fgx_stream_t stream) {
    return fgx_conv_gather_gemm_stream_act_mask(dtype, src, panel, bias, order, tile_code, plan_seg, plan_idx, plan_band, plan_rows,
                                                n, n_src, K, cols, V, tile_rows, tile_cols, slab_bytes, item_at, max_groups,
                                                activation, out, nullptr, stream);
}

extern "C" int fgx_conv_gather_gemm_stream_act_mask(int dtype, const void* src, const void* panel, const void* bias,
                                                    const int64_t* order, const int32_t* tile_code, const int32_t* plan_seg,
                                                    const uint32_t* plan_idx, const uint32_t* plan_band, size_t plan_rows,
                                                    size_t n, size_t n_src, int K, int cols, int V,
                                                    int tile_rows, int tile_cols, int slab_bytes, const uint32_t* item_at,
                                                    int max_groups, int activation, void* out, uint8_t* relu_mask,
                                                    fgx_stream_t stream) {
    FGX_CHECK_ARG(activation == FGX_ACT_NONE || activation == FGX_ACT_RELU, "fgx_conv_gather_gemm_stream: unknown activation %d", activation);
    FGX_CHECK_ARG(relu_mask == nullptr || (activation == FGX_ACT_RELU && dtype != FGX_F32 && cols % 8 == 0),
                  "fgx_conv_gather_gemm_stream: a ReLU mask needs the ReLU epilogue, a 16-bit type and a multiple of 8 columns (got %d)", cols);
    const int act = activation;
    FGX_CHECK_ARG(dtype == FGX_F16 || dtype == FGX_BF16 || dtype == FGX_F32, "fgx_conv_gather_gemm_stream: unknown dtype %d", dtype);
    FGX_CHECK_ARG(K > 0 && cols > 0 && V >= 1 && V <= 32, "fgx_conv_gather_gemm_stream: bad shape K=%d cols=%d V=%d", K, cols, V);
    if (n == 0) return FGX_OK;
    const int es = dtype == FGX_F32 ? 4 : 2;
    FGX_CHECK_ARG(((size_t)K * es) % 16 == 0, "fgx_conv_gather_gemm_stream: source row of %d elements is not a multiple of 16 bytes", K);
    FGX_CHECK_ARG(src && panel && order && plan_seg && tile_code && plan_idx && out, "fgx_conv_gather_gemm_stream: null buffer");
    FGX_CHECK_ARG((((uintptr_t)src | (uintptr_t)panel | (uintptr_t)plan_idx) & 15) == 0,
                  "fgx_conv_gather_gemm_stream: src, panel and plan_idx must be 16-byte aligned");
    FGX_CHECK_ARG(tile_rows > 0 && tile_cols > 0 && (slab_bytes == 64 || slab_bytes == 128), "fgx_conv_gather_gemm_stream: bad schedule");
    FGX_CHECK_ARG(plan_band == nullptr || tile_rows <= 1024, "fgx_conv_gather_gemm_stream: band masks cover tiles of at most 1024 rows");
    // 32-bit buffer offsets: every operand must stay below the out-of-range marker
    const size_t src_bytes = n_src * (size_t)K * es;
    const int cols_pad = (int)align_up((size_t)cols, (size_t)tile_cols);
    const size_t slabs = ((size_t)K * es + slab_bytes - 1) / slab_bytes;
    const size_t panel_bytes = (size_t)V * slabs * cols_pad * slab_bytes;
    if (src_bytes > kOobOffset || panel_bytes > kOobOffset || plan_rows * (size_t)tile_rows * 4 > kOobOffset || n * 8 > kOobOffset) {
        set_error("fgx_conv_gather_gemm_stream: an operand exceeds the 32-bit offset range (src %zu bytes); use fgx_conv_gather_gemm", src_bytes);
        return FGX_ERR_UNSUPPORTED;
    }
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case FGX_F16: return dispatch_stream<F16>(tile_rows, tile_cols, slab_bytes, src, panel, bias, order, plan_seg, tile_code, plan_idx, plan_band, plan_rows, n, n_src, K, cols, cols_pad, panel_bytes, item_at, max_groups, act, out, relu_mask, s);
        case FGX_BF16: return dispatch_stream<BF16>(tile_rows, tile_cols, slab_bytes, src, panel, bias, order, plan_seg, tile_code, plan_idx, plan_band, plan_rows, n, n_src, K, cols, cols_pad, panel_bytes, item_at, max_groups, act, out, relu_mask, s);
        default: return dispatch_stream<F32>(tile_rows, tile_cols, slab_bytes, src, panel, bias, order, plan_seg, tile_code, plan_idx, plan_band, plan_rows, n, n_src, K, cols, cols_pad, panel_bytes, item_at, max_groups, act, out, nullptr, s);
    }
}

namespace fgx {
bool stream_lds_fits(int tile_rows, int tile_cols, int slab_bytes, int cols) {
    if (cols <= 0 || tile_cols <= 0) return false;
    const size_t bias_bytes = align_up((size_t)cols, (size_t)tile_cols) * sizeof(float);
    size_t fixed = 0;       // (the ring sizes do not depend on the element type)
#define FGX_STREAM_TILE(BM, BN, WMv, WNv, CHv) \
    if (tile_rows == BM && tile_cols == BN && slab_bytes == CHv * 16) fixed = StreamCfg<F16, BM, BN, WMv, WNv, CHv>::fixed_lds;
    FGX_STREAM_TILE(256, 128, FGX_BIG_WAVES_M, 2, 8)
    FGX_STREAM_TILE(256, 64, 4, 2, 8)
    FGX_STREAM_TILE(128, 256, 2, 4, 8)      // few voxels, wide outputs: half the rows per tile pad less
    FGX_STREAM_TILE(256, 128, 4, 2, 4)
    FGX_STREAM_TILE(256, 64, 4, 2, 4)
    FGX_STREAM_TILE(256, 32, 8, 1, 4)
#undef FGX_STREAM_TILE
    return fixed != 0 && fixed + bias_bytes <= 160 * 1024;
}
}  // namespace fgx

extern "C" int fgx_conv_gather_gemm_stream_groups(int dtype, int cols, int tile_rows, int tile_cols, int slab_bytes,
                                                  int* groups) {
    FGX_CHECK_ARG(dtype == FGX_F16 || dtype == FGX_BF16 || dtype == FGX_F32, "fgx_conv_gather_gemm_stream_groups: unknown dtype %d", dtype);
    FGX_CHECK_ARG(groups != nullptr && cols > 0 && tile_cols > 0, "fgx_conv_gather_gemm_stream_groups: bad argument");
    const size_t bias_bytes = align_up((size_t)cols, (size_t)tile_cols) * sizeof(float);
#define FGX_STREAM_TILE(TAG, BM, BN, WMv, WNv, CHv)                                              \
    if (tile_rows == BM && tile_cols == BN && slab_bytes == CHv * 16)                            \
        return resident_groups<TAG, BM, BN, WMv, WNv, CHv>(StreamCfg<TAG, BM, BN, WMv, WNv, CHv>::fixed_lds + bias_bytes, groups);
#define FGX_STREAM_TILES(TAG)            \
    FGX_STREAM_TILE(TAG, 256, 128, FGX_BIG_WAVES_M, 2, 8) \
    FGX_STREAM_TILE(TAG, 256, 64, 4, 2, 8)  \
    FGX_STREAM_TILE(TAG, 128, 256, 2, 4, 8) \
    FGX_STREAM_TILE(TAG, 256, 128, 4, 2, 4) \
    FGX_STREAM_TILE(TAG, 256, 64, 4, 2, 4)  \
    FGX_STREAM_TILE(TAG, 256, 32, 8, 1, 4)
    if (dtype == FGX_F16) { FGX_STREAM_TILES(F16) }
    else if (dtype == FGX_BF16) { FGX_STREAM_TILES(BF16) }
    else { FGX_STREAM_TILES(F32) }
#undef FGX_STREAM_TILES
#undef FGX_STREAM_TILE
    set_error("fgx_conv_gather_gemm_stream_groups: no kernel for tile %dx%d with %d-byte slabs", tile_rows, tile_cols, slab_bytes);
    return FGX_ERR_UNSUPPORTED;
}
