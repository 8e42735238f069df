// Masked implicit GEMM (forward and dgrad) for submanifold sparse conv on gfx950.
//
//   out[sorted[r], :] = sum over offsets v present for row r of src[map[sorted[r], v], :] x panel_v (+ bias)
//
// One workgroup owns a tile of BM consecutive rows of the mask-sorted voxel order and BN output
// channels.  Offsets whose bit is clear in the tile's OR-mask are skipped altogether.  The remaining
// (offset, K-slab) steps stream through an S-stage ring in LDS: a stage holds the gathered source rows
// (A, BM x 64 bytes) and the matching weight-panel slice (B, BN x 64 bytes).  The neighbor indices of
// an offset (one column of the map, gathered through the sorted order) travel through a small ring of
// their own, S-1 steps ahead of the rows that need them.  All of it is moved by direct global->LDS loads
// (lane i of a wavefront deposits its data at LDS base + size * i), so several gathers are in flight
// per workgroup while the wavefronts multiply and nothing waits for an index table to be staged first.
// These loads are the only vector-memory operations in the main loop and every wavefront issues the
// same number per step (dummy loads where it has nothing to fetch), which makes the outstanding-load
// counter exact: "step k's rows and the indices for the next enqueue have landed" is
// s_waitcnt vmcnt((S-2) * loads_per_step), followed by one workgroup barrier per step.
//
// The gather is a per-lane choice of global address, so a missing neighbor (or a K tail) simply reads
// a block of zeros, and the bank-conflict swizzle of the 16-byte chunks is applied on the global side
// (lane -> which chunk of the row it fetches) since the LDS side of the load is fixed.
//
// The output tile is converted, passed through LDS and written as whole 16-byte pieces of a row.
//
// Each of the WAVES_M x WAVES_N wavefronts multiplies its (BM/WAVES_M) x (BN/WAVES_N) sub-tile with
// 32x32 MFMA instructions, accumulating in fp32.  Both operands are K-contiguous per row, and A and B
// fragments are read from LDS with the same (chunk, lane-group) -> k assignment, so the contraction is
// independent of how the hardware numbers k inside a fragment.
//
// dgrad is the same kernel: src = grad_output and a panel packed with the mirrored, transposed
// weight (fgx_pack_weight mode 1).
#include <atomic>

#include "gemm_device.h"

namespace fgx {
namespace {

// K-slab per row and step: 64 or 128 bytes (4 or 8 chunks of 16 bytes), a template parameter of the kernel
constexpr int kIdxSlots = 4;      // neighbor-index ring depth (>= row ring depth)

// 16 zero bytes every lane may read: missing neighbors, K tails, dummy loads past the last step
__device__ __attribute__((aligned(256))) unsigned char g_zero_block[256];
// the "no neighbor" word: index loads of rows past the end and dummy index loads read it
__device__ __attribute__((aligned(16))) const uint32_t g_empty_word[4] = {FGX_EMPTY32, FGX_EMPTY32, FGX_EMPTY32, FGX_EMPTY32};

// ------------------------------------------------------------------------------------------------
// Weight panels
// ------------------------------------------------------------------------------------------------
// panel[v][slab][col][k] with k in [0, SK); mode 0: w[col][v][slab*SK+k]; mode 1: w[slab*SK+k][V-1-v][col];
// mode 2: w[slab*SK+k][v][col] (input gradient through a separate backward map, no mirroring of v).
template <typename T>
__global__ void __launch_bounds__(256) pack_weight_kernel(const T* __restrict__ w, int Ci, int Co, int V, int mode,
                                                          int slab_bytes, int slabs, int cols_pad, T* __restrict__ panel) {
    const int SK = slab_bytes / (int)sizeof(T);
    const int K = mode == 0 ? Ci : Co;
    const int cols = mode == 0 ? Co : Ci;
    const size_t total = (size_t)V * slabs * cols_pad * SK;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        int k = (int)(i % SK);
        size_t t = i / SK;
        int col = (int)(t % cols_pad);
        t /= cols_pad;
        int slab = (int)(t % slabs);
        int v = (int)(t / slabs);
        int kk = slab * SK + k;
        T val = (T)0;
        if (kk < K && col < cols) {
            if (mode == 0) val = w[((size_t)col * V + v) * Ci + kk];
            else val = w[((size_t)kk * V + (mode == 1 ? V - 1 - v : v)) * Ci + col];
        }
        panel[i] = val;
    }
}

// The same panels for 16-bit types whose channel counts are multiples of 8, moved 16 bytes at a time.
//
// Forward panels copy runs: panel[v][slab][col][0, SK) is w[col][v][slab*SK, +SK), contiguous on both sides.  One thread
// per 16-byte piece; grid = (pieces of a (v, slab) plane / 256, slabs, V), so no index needs a division.
template <int SK>
__global__ void __launch_bounds__(256) pack_weight_rows_kernel(const uint16_t* __restrict__ w, int Ci, int Co, int V,
                                                               int cols_pad, uint16_t* __restrict__ panel) {
    constexpr int PIECES = SK / 8;                          // 16-byte pieces per (col, slab) run
    const int piece = blockIdx.x * 256 + threadIdx.x;       // inside the (v, slab) plane
    if (piece >= cols_pad * PIECES) return;
    const int col = piece / PIECES, kk = blockIdx.y * SK + (piece % PIECES) * 8, v = blockIdx.z;
    uint4 val = make_uint4(0u, 0u, 0u, 0u);
    if (col < Co && kk < Ci) val = *reinterpret_cast<const uint4*>(w + ((size_t)col * V + v) * Ci + kk);
    *reinterpret_cast<uint4*>(panel + (((size_t)v * gridDim.y + blockIdx.y) * cols_pad) * SK + (size_t)piece * 8) = val;
}

// Input-gradient panels transpose: panel[v][slab][col][k] is w[slab*SK + k][v'][col] (v' = V-1-v when the offsets are
// mirrored), contiguous along col in w and along k in the panel.  A workgroup moves one SK x 32 tile through LDS:
// 16-byte reads along col, 2-byte LDS stores into the transposed tile, 16-byte LDS reads and stores along k.
template <int SK>
__global__ void __launch_bounds__(256) pack_weight_transpose_kernel(const uint16_t* __restrict__ w, int Ci, int Co, int V,
                                                                    int mirror, int cols_pad, uint16_t* __restrict__ panel) {
    constexpr int PITCH = SK + 8;                           // halfwords; keeps every row 16-byte aligned
    __shared__ __attribute__((aligned(16))) uint16_t tile[32 * PITCH];
    const int col0 = blockIdx.x * 32, slab = blockIdx.y, v = blockIdx.z;
    const int vsrc = mirror ? V - 1 - v : v;
    const int t = threadIdx.x;
    if (t < SK * 4) {
        const int r = t >> 2, c8 = (t & 3) * 8;             // row of the tile (a k value), first of 8 columns
        const int kk = slab * SK + r, col = col0 + c8;
        uint4 val = make_uint4(0u, 0u, 0u, 0u);
        if (kk < Co && col < Ci) val = *reinterpret_cast<const uint4*>(w + ((size_t)kk * V + vsrc) * Ci + col);
        const uint32_t words[4] = {val.x, val.y, val.z, val.w};
#pragma unroll
        for (int j = 0; j < 8; ++j) tile[(c8 + j) * PITCH + r] = (uint16_t)(words[j >> 1] >> ((j & 1) * 16));
    }
    __syncthreads();
    constexpr int PIECES = SK / 8;
    if (t < 32 * PIECES) {
        const int c = t / PIECES, k8 = (t % PIECES) * 8;
        const uint4 val = *reinterpret_cast<const uint4*>(tile + c * PITCH + k8);
        *reinterpret_cast<uint4*>(panel + ((((size_t)v * gridDim.y + slab) * cols_pad) + col0 + c) * SK + k8) = val;
    }
}

// ------------------------------------------------------------------------------------------------
// Gather GEMM
// ------------------------------------------------------------------------------------------------
template <typename Tag, int BM, int BN, int WAVES_M, int WAVES_N, int S, int CH>
struct GemmCfg {
    using T = typename Tag::type;
    static constexpr int ES = (int)sizeof(T);
    static constexpr int NW = WAVES_M * WAVES_N;
    static constexpr int NT = 64 * NW;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int TM = WM / 32, TN = WN / 32;
    static constexpr int SLAB = CH * 16;                             // bytes of K per row and step
    static constexpr int SK = SLAB / ES;
    static constexpr int ROWS_PER_INST = 64 / CH;                    // slab rows one wave-wide load covers
    static constexpr int A_INST = BM / ROWS_PER_INST, B_INST = BN / ROWS_PER_INST;
    static constexpr int A_PER = (A_INST + NW - 1) / NW, B_PER = (B_INST + NW - 1) / NW;  // row loads per wavefront and step
    static constexpr int IDX_INST = (BM + 63) / 64;                  // wave-wide loads per index column
    static constexpr int LPS = A_PER + B_PER + 1;                    // + one index load
    static constexpr int STAGE_BYTES = (BM + BN) * SLAB;
    static constexpr int IDX_SLOT_BYTES = IDX_INST * 256;
    static constexpr int OUT_PITCH = WN * ES + 16;                   // epilogue band: 32 rows of a wave tile
    static constexpr int OUT_BAND_BYTES = 32 * OUT_PITCH;
    static constexpr int RING_BYTES = S * STAGE_BYTES > NW * OUT_BAND_BYTES ? S * STAGE_BYTES : NW * OUT_BAND_BYTES;
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert(BM % ROWS_PER_INST == 0 && BN % ROWS_PER_INST == 0, "tile must be whole wave-wide loads");
    static_assert((S - 2) * LPS < 64 && S >= 3 && S <= kIdxSlots, "ring depth out of range");
    static_assert(CH == 4 || CH == 8, "slab must be 64 or 128 bytes");
    static_assert((WN * ES) % 16 == 0, "a band row must be whole 16-byte pieces");
    static constexpr size_t lds_bytes = (size_t)RING_BYTES + (size_t)kIdxSlots * IDX_SLOT_BYTES + 1024 + (size_t)BM * 4 + 32 * 4;
};

template <typename Tag, int BM, int BN, int WAVES_M, int WAVES_N, int S, int CH>
__global__ void __launch_bounds__(64 * WAVES_M * WAVES_N)
gather_gemm_kernel(const typename Tag::type* __restrict__ src, const typename Tag::type* __restrict__ panel,
                   const typename Tag::type* __restrict__ bias, const uint32_t* __restrict__ map,
                   const int64_t* __restrict__ sorted_idx, const int32_t* __restrict__ tile_code, uint32_t n, int K,
                   int cols, int cols_pad, int V, int splitk, unsigned row_tiles, unsigned col_tiles,
                   float* __restrict__ partial, int act, typename Tag::type* __restrict__ out,
                   uint8_t* __restrict__ relu_mask) {
    using C = GemmCfg<Tag, BM, BN, WAVES_M, WAVES_N, S, CH>;
    using T = typename Tag::type;
    constexpr int NT = C::NT;
    constexpr int kSlabBytes = C::SLAB, kChunks = CH;

    // XCD-aware tile order: workgroups are dealt round-robin to the 8 XCDs, so give each XCD a
    // contiguous run of tiles (all column tiles of a row tile share their gathered rows -> same L2).
    const unsigned total_tiles = row_tiles * col_tiles;
    const unsigned per_xcd = (total_tiles + kXcds - 1) / kXcds;
    const unsigned logical = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
    if (logical >= total_tiles) return;
    const unsigned row_tile = logical / col_tiles;
    const unsigned col_tile = logical % col_tiles;
    const int kid = blockIdx.y;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    unsigned char* ring = lds_raw;                                        // [S][A: BM x 64 | B: BN x 64]; epilogue bands later
    unsigned char* idx_ring = ring + C::RING_BYTES;                       // [kIdxSlots][BM] neighbor rows of one offset
    unsigned char* dump = idx_ring + kIdxSlots * C::IDX_SLOT_BYTES;       // 1 KiB sink of surplus loads
    uint32_t* row_lds = (uint32_t*)(dump + 1024);                         // [BM] output row or EMPTY
    int* v_lds = (int*)(row_lds + BM);                                    // [32] offsets present in this tile

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const uint32_t code = (uint32_t)tile_code[row_tile];
    const int nv = __popc(code);
    const int slabs = (K + C::SK - 1) / C::SK;
    const int steps_total = nv * slabs;
    const int step_lo = (int)(((long long)steps_total * kid + splitk - 1) / splitk);
    const int step_hi = (int)(((long long)steps_total * (kid + 1) + splitk - 1) / splitk);

    // ---- the tile's output rows; every wavefront also keeps the rows whose indices it will fetch ----
    const int idx_inst = wave % C::IDX_INST;
    const bool idx_owner = wave < C::IDX_INST;               // the other wavefronts only issue dummy index loads
    const int idx_row = idx_inst * 64 + lane;
    uint32_t my_row = FGX_EMPTY32;
    {
        const size_t gr = (size_t)row_tile * BM + idx_row;
        if (idx_row < BM && gr < n) my_row = (uint32_t)sorted_idx[gr];
    }
    for (int r = tid; r < BM; r += NT) {
        size_t gr = (size_t)row_tile * BM + r;
        row_lds[r] = gr < n ? (uint32_t)sorted_idx[gr] : FGX_EMPTY32;
    }
    if (tid == 0) {
        uint32_t c = code;
        int i = 0;
        while (c) {
            v_lds[i++] = __ffs((int)c) - 1;
            c &= c - 1;
        }
    }
    __syncthreads();   // also drains every outstanding vector-memory load: the counter starts at zero below

    f32x16 acc[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const size_t row_bytes = (size_t)K * sizeof(T);
    const unsigned char* src_b = (const unsigned char*)src;
    const unsigned char* panel_b = (const unsigned char*)panel;
    const unsigned char* zero_b = g_zero_block;
    const int sub_row = lane / kChunks, pch = lane % kChunks;
    const bool ragged = (row_bytes % kSlabBytes) != 0;   // last slab of a row is partly past the row end

    // ---- index stream: one load per wavefront and step; a real one when a new offset comes into view ----
    const uint32_t* my_map = my_row != FGX_EMPTY32 ? map + (size_t)my_row * V : nullptr;
    int ix_step = step_lo, ix_vi = slabs > 0 ? step_lo / slabs : 0, ix_slab = step_lo - ix_vi * slabs;
    int ix_done = -1;                                      // last offset slot whose load has been enqueued
    auto issue_idx = [&]() {
        const bool need = ix_step < step_hi && ix_vi > ix_done;      // wave-uniform
        const uint32_t* p = g_empty_word;
        unsigned char* dst = dump;
        if (need) {
            if (idx_owner) {
                const int v = v_lds[ix_vi];
                if (my_map != nullptr) p = my_map + v;
                dst = idx_ring + (ix_vi % kIdxSlots) * C::IDX_SLOT_BYTES + idx_inst * 256;
            }
            ix_done = ix_vi;
        }
        __builtin_amdgcn_global_load_lds(FGX_GLOBAL_PTR(p), FGX_LDS_PTR(dst), 4, 0, 0);
        ++ix_step;
        if (++ix_slab == slabs) {
            ix_slab = 0;
            ++ix_vi;
        }
    };

    // ---- row stream: runs S-1 steps ahead of the multiply stream and keeps per-lane source pointers that
    // advance by one slab per step; they are re-derived only when the offset changes ----
    int a_row[C::A_PER], a_choff[C::A_PER], a_inc[C::A_PER], b_off[C::B_PER];
    bool a_mine[C::A_PER], b_mine[C::B_PER];
    const unsigned char* a_ptr[C::A_PER];
#pragma unroll
    for (int i = 0; i < C::A_PER; ++i) {
        const int inst = i * C::NW + wave;
        a_mine[i] = C::A_INST % C::NW == 0 || inst < C::A_INST;          // wave-uniform
        a_row[i] = (a_mine[i] ? inst : 0) * C::ROWS_PER_INST + sub_row;
        a_choff[i] = (pch ^ swz_key<CH>(a_row[i])) << 4;
        a_ptr[i] = zero_b;
        a_inc[i] = 0;
    }
#pragma unroll
    for (int i = 0; i < C::B_PER; ++i) {
        const int inst = i * C::NW + wave;
        b_mine[i] = C::B_INST % C::NW == 0 || inst < C::B_INST;          // wave-uniform
        const int col = (b_mine[i] ? inst : 0) * C::ROWS_PER_INST + sub_row;
        b_off[i] = col * kSlabBytes + ((pch ^ swz_key<CH>(col)) << 4);
    }
    const size_t b_slab_stride = (size_t)cols_pad * kSlabBytes;
    const unsigned char* b_ptr = zero_b;   // panel slice of the row stream's (offset, slab), column tile applied
    size_t b_inc = 0;
    int is_step = step_lo;                 // next step to enqueue
    int is_vi = slabs > 0 ? step_lo / slabs : 0;
    int is_slab = step_lo - is_vi * slabs;
    int is_stage = 0;
    bool is_fresh = true;                  // pointers must be (re)derived before the next enqueue

    auto issue_rows = [&]() {
        unsigned char* stage = ring + is_stage * C::STAGE_BYTES;
        if (is_fresh) {                    // wave-uniform: first call, offset change, or running off the end
            const bool live = is_step < step_hi;
            const int v = v_lds[live ? is_vi : 0];
            const uint32_t* slot = (const uint32_t*)(idx_ring + ((live ? is_vi : 0) % kIdxSlots) * C::IDX_SLOT_BYTES);
#pragma unroll
            for (int i = 0; i < C::A_PER; ++i) {
                const uint32_t m = slot[a_row[i]];
                const bool real = live && a_mine[i] && m != FGX_EMPTY32;
                const size_t off = real ? (size_t)m * row_bytes + (size_t)(is_slab * kSlabBytes + a_choff[i]) : (size_t)0;
                a_ptr[i] = real ? src_b + off : zero_b;
                a_inc[i] = real ? kSlabBytes : 0;
            }
            b_ptr = live ? panel_b + (((size_t)v * slabs + is_slab) * cols_pad + (size_t)col_tile * BN) * kSlabBytes : zero_b;
            b_inc = live ? b_slab_stride : 0;
            is_fresh = false;
        }
        const bool tail = ragged && is_slab == slabs - 1;   // wave-uniform
#pragma unroll
        for (int i = 0; i < C::A_PER; ++i) {
            const unsigned char* p = a_ptr[i];
            if (tail) p = (size_t)(is_slab * kSlabBytes + a_choff[i]) < row_bytes ? p : zero_b;
            unsigned char* dst = a_mine[i] ? stage + (i * C::NW + wave) * 1024 : dump;
            __builtin_amdgcn_global_load_lds(FGX_GLOBAL_PTR(p), FGX_LDS_PTR(dst), 16, 0, 0);
            a_ptr[i] += a_inc[i];
        }
#pragma unroll
        for (int i = 0; i < C::B_PER; ++i) {
            const unsigned char* p = (b_inc != 0 && b_mine[i]) ? b_ptr + b_off[i] : zero_b;
            unsigned char* dst = b_mine[i] ? stage + BM * kSlabBytes + (i * C::NW + wave) * 1024 : dump;
            __builtin_amdgcn_global_load_lds(FGX_GLOBAL_PTR(p), FGX_LDS_PTR(dst), 16, 0, 0);
        }
        b_ptr += b_inc;
        ++is_step;
        is_stage = is_stage + 1 == S ? 0 : is_stage + 1;
        if (++is_slab == slabs) {
            is_slab = 0;
            ++is_vi;
            is_fresh = true;
        }
        if (is_step == step_hi) is_fresh = true;
    };

    // ---- prologue: indices of the first S-1 steps, then S-1 enqueue rounds ----
#pragma unroll
    for (int s = 0; s < S - 1; ++s) issue_idx();
    wait_vmcnt<0>();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int s = 0; s < S - 1; ++s) {
        issue_rows();
        issue_idx();
    }

    const int g = lane >> 5;        // lane group inside the MFMA fragment
    const int l32 = lane & 31;
    int a_frag[kChunks / 2][C::TM], b_frag[kChunks / 2][C::TN];   // byte offsets of this lane's fragments in a stage
#pragma unroll
    for (int kk = 0; kk < kChunks / 2; ++kk) {
#pragma unroll
        for (int i = 0; i < C::TM; ++i) a_frag[kk][i] = swz<CH>(wave_m * C::WM + i * 32 + l32, kk * 2 + g);
#pragma unroll
        for (int j = 0; j < C::TN; ++j) b_frag[kk][j] = BM * kSlabBytes + swz<CH>(wave_n * C::WN + j * 32 + l32, kk * 2 + g);
    }
    int cur_stage = 0;
    for (int step = step_lo; step < step_hi; ++step) {
        // rows of `step` and the indices the next enqueue needs are older than the (S-2) * LPS newest loads
        wait_vmcnt<(S - 2) * C::LPS>();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();      // everybody's loads landed; the stage read in the previous step is free again
        asm volatile("" ::: "memory");
        issue_rows();
        issue_idx();
        const unsigned char* cur = ring + cur_stage * C::STAGE_BYTES;
        cur_stage = cur_stage + 1 == S ? 0 : cur_stage + 1;
        u32x4 af[kChunks / 2][C::TM], bf[kChunks / 2][C::TN];
#pragma unroll
        for (int kk = 0; kk < kChunks / 2; ++kk) {
#pragma unroll
            for (int i = 0; i < C::TM; ++i) af[kk][i] = *(const u32x4*)(cur + a_frag[kk][i]);
#pragma unroll
            for (int j = 0; j < C::TN; ++j) bf[kk][j] = *(const u32x4*)(cur + b_frag[kk][j]);
        }
#pragma unroll
        for (int kk = 0; kk < kChunks / 2; ++kk)
#pragma unroll
            for (int i = 0; i < C::TM; ++i)
#pragma unroll
                for (int j = 0; j < C::TN; ++j) mma<Tag>(acc[i][j], af[kk][i], bf[kk][j]);
    }
    wait_vmcnt<0>();   // the trailing dummy loads
    __syncthreads();   // the ring is reused below

    // ---- epilogue.  32x32 accumulator tile: element e of lane l is row 8*(e/4) + 4*(l/32) + e%4, column l%32. ----
    if (splitk > 1) {
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
            const int col = (int)col_tile * BN + wave_n * C::WN + j * 32 + l32;
            if (col >= cols) continue;
            const float bv = (bias != nullptr && kid == 0) ? to_float<T>(bias[col]) : 0.f;
#pragma unroll
            for (int i = 0; i < C::TM; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int r = wave_m * C::WM + i * 32 + (e >> 2) * 8 + g * 4 + (e & 3);
                    const uint32_t orow = row_lds[r];
                    if (orow != FGX_EMPTY32) partial[((size_t)kid * n + orow) * cols + col] = acc[i][j][e] + bv;
                }
        }
        return;
    }
    // One 32-row band of the wave tile at a time: add the bias, convert, park the band in LDS (each wavefront has
    // its own area), then write whole 16-byte pieces of output rows.
    unsigned char* band = ring + wave * C::OUT_BAND_BYTES;
    float bv[C::TN];
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
        const int col = (int)col_tile * BN + wave_n * C::WN + j * 32 + l32;
        bv[j] = (bias != nullptr && col < cols) ? to_float<T>(bias[col]) : 0.f;
    }
    constexpr int PIECES = C::WN * C::ES / 16;                // 16-byte pieces per band row
    constexpr int ROWS_PER_PASS = 64 / PIECES;
    const int col0 = (int)col_tile * BN + wave_n * C::WN;     // first output column of the wave tile
    const bool vec_ok = (cols * C::ES) % 16 == 0;             // output rows start on 16-byte boundaries
#pragma unroll
    for (int i = 0; i < C::TM; ++i) {
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int r = (e >> 2) * 8 + g * 4 + (e & 3);
                *(T*)(band + r * C::OUT_PITCH + (j * 32 + l32) * C::ES) = from_float<T>(activate(acc[i][j][e] + bv[j], act));
            }
        // same wavefront wrote and reads: program order inside the wavefront suffices for LDS
#pragma unroll
        for (int pass = 0; pass < 32 / ROWS_PER_PASS; ++pass) {
            const int r = pass * ROWS_PER_PASS + lane / PIECES;
            const int piece = lane % PIECES;
            const uint32_t orow = row_lds[wave_m * C::WM + i * 32 + r];
            const int col = col0 + piece * (16 / C::ES);
            if (orow == FGX_EMPTY32 || col >= cols) continue;
            const unsigned char* sp = band + r * C::OUT_PITCH + piece * 16;
            T* dp = out + (size_t)orow * cols + col;
            if (vec_ok && col + 16 / C::ES <= cols) {
                const u32x4 piece16 = *(const u32x4*)sp;
                *(u32x4*)dp = piece16;
                // one bit per output for the activation's derivative (16-bit types, whole pieces only: the host passes a
                // mask for such shapes alone)
                if (C::ES == 2 && relu_mask != nullptr)
                    relu_mask[((size_t)orow * cols + col) >> 3] = (uint8_t)positive_bits16<PositiveLimit<T>::value>(piece16);
            } else {
                for (int t = 0; t < 16 / C::ES && col + t < cols; ++t) dp[t] = ((const T*)sp)[t];
            }
        }
    }
}

// out[i] = act(sum_s partial[s][i])   (slice 0 carries the bias).  relu_mask != nullptr (numel a multiple of 8): bit i says
// whether out[i] > 0 -- a wavefront holds 64 consecutive i, one ballot gives their bits and every eighth lane writes a byte.
template <typename T>
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float* __restrict__ partial, int splitk, size_t numel,
                                                            int act, T* __restrict__ out, uint8_t* __restrict__ relu_mask) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < numel; i += (size_t)gridDim.x * 256) {
        float s = 0.f;
        for (int k = 0; k < splitk; ++k) s += partial[(size_t)k * numel + i];
        const T rounded = from_float<T>(activate(s, act));
        out[i] = rounded;
        if (relu_mask != nullptr) {
            const unsigned long long positive = __ballot(to_float<T>(rounded) > 0.f);
            const unsigned lane = threadIdx.x & 63u;
            if ((lane & 7u) == 0u) relu_mask[i >> 3] = (uint8_t)(positive >> lane);
        }
    }
}

// out[8 i .. 8 i + 7] = grad[...] where bit t of mask[i] is set, else 0 (16-bit elements: one 16-byte piece per lane)
__global__ void __launch_bounds__(256) relu_mask_apply_kernel(const u32x4* __restrict__ grad, const uint8_t* __restrict__ mask,
                                                              size_t pieces, u32x4* __restrict__ out) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < pieces; i += (size_t)gridDim.x * 256) {
        const uint32_t m = mask[i];
        u32x4 v = __builtin_nontemporal_load(grad + i);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const uint32_t keep = ((m >> (2 * w)) & 1u ? 0x0000FFFFu : 0u) | ((m >> (2 * w + 1)) & 1u ? 0xFFFF0000u : 0u);
            v[w] &= keep;
        }
        __builtin_nontemporal_store(v, out + i);
    }
}

// Column sums with fp32 accumulation.  Stage 1: kColsumSlices blocks each sum a contiguous slice of rows with
// 16-byte loads (a thread owns VEC adjacent columns, the block's row lanes are added through LDS); stage 2 adds
// the slices in a fixed order, so the result is deterministic.
constexpr int kColsumSlices = 1024;
template <typename T, int VEC>
__global__ void __launch_bounds__(256) colsum_partial_kernel(const T* __restrict__ x, size_t n, int cols,
                                                             float* __restrict__ partial) {
    __shared__ float red[256 * VEC];
    const int groups = (cols + VEC - 1) / VEC;
    const int tpr = groups < 256 ? groups : 256;    // threads across one row
    const int lanes = 256 / tpr;                    // row lanes of the block
    const int cg0 = threadIdx.x % tpr, rl = threadIdx.x / tpr;
    const size_t per = (n + gridDim.x - 1) / gridDim.x;
    const size_t r0 = (size_t)blockIdx.x * per;
    const size_t r1 = r0 + per < n ? r0 + per : n;
    for (int cg = cg0; cg < groups; cg += tpr) {
        float acc[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
        if (rl < lanes) {
            size_t r = r0 + rl;
            if constexpr (VEC > 1) {
                // four rows per trip: four independent 16-byte loads in flight, added in row order
                for (; r + 3 * (size_t)lanes < r1; r += 4 * (size_t)lanes) {
                    u32x4 raw[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) raw[q] = *(const u32x4*)(x + (r + (size_t)q * lanes) * cols + (size_t)cg * VEC);
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const T* v = (const T*)&raw[q];
#pragma unroll
                        for (int e = 0; e < VEC; ++e) acc[e] += to_float<T>(v[e]);
                    }
                }
            }
            for (; r < r1; r += lanes) {
                const T* src = x + r * cols + (size_t)cg * VEC;
                if constexpr (VEC == 1) {
                    acc[0] += to_float<T>(src[0]);
                } else {
                    u32x4 raw = *(const u32x4*)src;
                    const T* v = (const T*)&raw;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[e] += to_float<T>(v[e]);
                }
            }
        }
        if (lanes > 1) {   // uniform over the block: groups <= 128, a single pass of the cg loop
#pragma unroll
            for (int e = 0; e < VEC; ++e) red[threadIdx.x * VEC + e] = acc[e];
            __syncthreads();
            if (rl == 0) {
                for (int l = 1; l < lanes; ++l)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[e] += red[(l * tpr + cg0) * VEC + e];
            }
        }
        if (rl == 0) {
#pragma unroll
            for (int e = 0; e < VEC; ++e)
                if (cg * VEC + e < cols) partial[(size_t)blockIdx.x * cols + cg * VEC + e] = acc[e];
        }
    }
}
// 16 columns per block, 16 threads per column each adding a sixteenth of the slices, then a fixed-order LDS sum
template <typename T>
__global__ void __launch_bounds__(256) colsum_final_kernel(const float* __restrict__ partial, unsigned slices, int cols,
                                                           T* __restrict__ out) {
    __shared__ float red[256];
    const int c = blockIdx.x * 16 + (threadIdx.x & 15);
    const int part = threadIdx.x >> 4;
    float s = 0.f;
    if (c < cols) {
        unsigned b = part;
        for (; b + 7 * 16 < slices; b += 8 * 16) {     // eight independent loads in flight, added in slice order
            float x[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) x[q] = partial[(size_t)(b + q * 16) * cols + c];
#pragma unroll
            for (int q = 0; q < 8; ++q) s += x[q];
        }
        for (; b < slices; b += 16) s += partial[(size_t)b * cols + c];
    }
    red[threadIdx.x] = s;
    __syncthreads();
    if (part == 0 && c < cols) {
        float t = 0.f;
#pragma unroll
        for (int p = 0; p < 16; ++p) t += red[p * 16 + threadIdx.x];
        out[c] = from_float<T>(t);
    }
}

int elem_size(int dtype) { return dtype == FGX_F32 ? 4 : 2; }
bool dtype_ok(int dtype) { return dtype == FGX_F16 || dtype == FGX_BF16 || dtype == FGX_F32; }

template <typename Tag, int BM, int BN, int WAVES_M, int WAVES_N, int S, int CH>
int launch_gemm(const void* src, const void* panel, const void* bias, const uint32_t* map, const int64_t* sorted_idx,
                const int32_t* tile_code, size_t n, int K, int cols, int cols_pad, int V, int splitk, void* scratch,
                int act, void* out, uint8_t* relu_mask, hipStream_t s) {
    using C = GemmCfg<Tag, BM, BN, WAVES_M, WAVES_N, S, CH>;
    using T = typename Tag::type;
    auto kern = gather_gemm_kernel<Tag, BM, BN, WAVES_M, WAVES_N, S, CH>;
    constexpr size_t lds = C::lds_bytes;
    static_assert(lds <= 160 * 1024, "tile does not fit the 160 KiB LDS");
    static thread_local bool lds_raised = false;   // raise the dynamic LDS limit once per thread and instantiation
    if (lds > 64 * 1024 && !lds_raised) {
        FGX_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        lds_raised = true;
    }
    const unsigned row_tiles = cdiv(n, BM), col_tiles = cdiv(cols, BN);
    const unsigned total = row_tiles * col_tiles;
    const unsigned grid_x = cdiv(total, kXcds) * kXcds;
    dim3 grid(grid_x, splitk, 1);
    kern<<<grid, C::NT, lds, s>>>((const T*)src, (const T*)panel, (const T*)bias, map, sorted_idx, tile_code, (uint32_t)n, K,
                                  cols, cols_pad, V, splitk, row_tiles, col_tiles, (float*)scratch, act, (T*)out,
                                  splitk > 1 ? nullptr : relu_mask);
    FGX_CHECK_LAUNCH("fgx_conv_gather_gemm");
    if (splitk > 1) {
        size_t numel = n * (size_t)cols;
        unsigned g = cdiv(numel, 256);
        if (g > 65536u) g = 65536u;
        splitk_reduce_kernel<T><<<g, 256, 0, s>>>((const float*)scratch, splitk, numel, act, (T*)out, relu_mask);
        FGX_CHECK_LAUNCH("fgx_conv_gather_gemm(reduce)");
    }
    return FGX_OK;
}

template <typename Tag>
int dispatch_tile(int tile_rows, int tile_cols, int slab_bytes, const void* src, const void* panel, const void* bias,
                  const uint32_t* map, const int64_t* sorted_idx, const int32_t* tile_code, size_t n, int K, int cols,
                  int cols_pad, int V, int splitk, void* scratch, int act, void* out, uint8_t* relu_mask, hipStream_t s) {
#define FGX_TILE(BM, BN, WMv, WNv, Sv, CHv)                                                                        \
    if (tile_rows == BM && tile_cols == BN && slab_bytes == CHv * 16)                                              \
        return launch_gemm<Tag, BM, BN, WMv, WNv, Sv, CHv>(src, panel, bias, map, sorted_idx, tile_code, n, K, cols, \
                                                           cols_pad, V, splitk, scratch, act, out, relu_mask, s);
    FGX_TILE(256, 128, 2, 2, 3, 4)
    FGX_TILE(256, 128, 4, 2, 3, 8)
    FGX_TILE(128, 128, 2, 2, 3, 4)
    FGX_TILE(128, 64, 2, 2, 3, 4)
    FGX_TILE(128, 32, 4, 1, 3, 4)
    FGX_TILE(64, 64, 2, 2, 3, 4)
    FGX_TILE(64, 32, 2, 1, 3, 4)
    FGX_TILE(32, 32, 1, 1, 3, 4)
#undef FGX_TILE
    set_error("fgx_conv_gather_gemm: no kernel for tile %dx%d with %d-byte slabs", tile_rows, tile_cols, slab_bytes);
    return FGX_ERR_UNSUPPORTED;
}

// both column-sum kernels on `s`, partial sums in `scratch` (kColsumSlices x cols floats)
int colsum_launch(int dtype, const void* x, size_t n, int cols, float* scratch, void* out, hipStream_t s) {
    unsigned slices = n ? (unsigned)((n + 255) / 256) : 0u;     // at least 256 rows per slice
    if (slices > (unsigned)kColsumSlices) slices = kColsumSlices;
    const unsigned gfin = cdiv(cols, 16);
    const int es = elem_size(dtype);
    const bool vec = ((size_t)cols * es) % 16 == 0 && ((uintptr_t)x & 15) == 0;
#define FGX_COLSUM(T, VEC)                                                                                  \
    do {                                                                                                    \
        if (slices) colsum_partial_kernel<T, VEC><<<slices, 256, 0, s>>>((const T*)x, n, cols, scratch);    \
        colsum_final_kernel<T><<<gfin, 256, 0, s>>>((const float*)scratch, slices, cols, (T*)out);          \
    } while (0)
    if (dtype == FGX_F16) { if (vec) FGX_COLSUM(_Float16, 8); else FGX_COLSUM(_Float16, 1); }
    else if (dtype == FGX_BF16) { if (vec) FGX_COLSUM(__bf16, 8); else FGX_COLSUM(__bf16, 1); }
    else { if (vec) FGX_COLSUM(float, 4); else FGX_COLSUM(float, 1); }
#undef FGX_COLSUM
    FGX_CHECK_LAUNCH("fgx_colsum");
    return FGX_OK;
}

constexpr int kStaticColsumCols = 2048;     // widest tensor fgx_colsum_static serves
constexpr int kMaxDevices = 64;

}  // namespace
}  // namespace fgx

// Scratch of fgx_colsum_static: the partial sums of the column sum for up to kStaticColsumCols columns (8 MiB), held
// by every GPU the library runs on until the process ends.  In host code this name is only a handle for
// hipGetSymbolAddress: kernels and copies are given the device address found there (one per device), never the name.
static __device__ __align__(256) float g_static_colsum_scratch[(size_t)fgx::kColsumSlices * fgx::kStaticColsumCols];
static std::atomic<float*> g_static_colsum_ptr[fgx::kMaxDevices];

using namespace fgx;

extern "C" {

size_t fgx_weight_panel_bytes(int dtype, int mode, int Ci, int Co, int V, int slab_bytes, int col_pad) {
    if (!dtype_ok(dtype) || Ci <= 0 || Co <= 0 || V <= 0 || col_pad <= 0 || (slab_bytes != 64 && slab_bytes != 128)) return 0;
    const int K = mode == 0 ? Ci : Co, cols = mode == 0 ? Co : Ci;
    const int es = elem_size(dtype), SK = slab_bytes / es;
    const size_t slabs = (size_t)(K + SK - 1) / SK;
    const size_t cols_pad = align_up((size_t)cols, (size_t)col_pad);
    return (size_t)V * slabs * cols_pad * slab_bytes;
}

int fgx_pack_weight(int dtype, int mode, const void* weight, int Ci, int Co, int V, int slab_bytes, int col_pad,
                    void* panel, fgx_stream_t stream) {
    FGX_CHECK_ARG(dtype_ok(dtype), "fgx_pack_weight: unknown dtype %d", dtype);
    FGX_CHECK_ARG(mode >= 0 && mode <= 2, "fgx_pack_weight: mode must be 0 (forward), 1 (dgrad, mirrored offsets) or 2 (dgrad)");
    FGX_CHECK_ARG(Ci > 0 && Co > 0 && V > 0, "fgx_pack_weight: bad shape Ci=%d Co=%d V=%d", Ci, Co, V);
    FGX_CHECK_ARG(col_pad > 0 && col_pad % 32 == 0, "fgx_pack_weight: col_pad must be a positive multiple of 32");
    FGX_CHECK_ARG(slab_bytes == 64 || slab_bytes == 128, "fgx_pack_weight: slab_bytes must be 64 or 128, got %d", slab_bytes);
    FGX_CHECK_ARG(weight && panel, "fgx_pack_weight: null buffer");
    const int K = mode == 0 ? Ci : Co, cols = mode == 0 ? Co : Ci;
    const int es = elem_size(dtype), SK = slab_bytes / es;
    const int slabs = (K + SK - 1) / SK;
    const int cols_pad = (int)align_up((size_t)cols, (size_t)col_pad);
    const size_t total = (size_t)V * slabs * cols_pad * SK;
    unsigned grid = cdiv(total, 256);
    if (grid > 32768u) grid = 32768u;
    hipStream_t s = (hipStream_t)stream;
    const bool wide = es == 2 && Ci % 8 == 0 && Co % 8 == 0 && (((uintptr_t)weight | (uintptr_t)panel) & 15) == 0 &&
                      slabs <= 65535 && V <= 65535;
    if (wide) {
        const uint16_t* w16 = (const uint16_t*)weight;
        uint16_t* p16 = (uint16_t*)panel;
        if (mode == 0) {
            const dim3 g(cdiv((size_t)cols_pad * (SK / 8), 256), slabs, V);
            if (SK == 64) pack_weight_rows_kernel<64><<<g, 256, 0, s>>>(w16, Ci, Co, V, cols_pad, p16);
            else pack_weight_rows_kernel<32><<<g, 256, 0, s>>>(w16, Ci, Co, V, cols_pad, p16);
        } else {
            const dim3 g(cols_pad / 32, slabs, V);
            if (SK == 64) pack_weight_transpose_kernel<64><<<g, 256, 0, s>>>(w16, Ci, Co, V, mode == 1, cols_pad, p16);
            else pack_weight_transpose_kernel<32><<<g, 256, 0, s>>>(w16, Ci, Co, V, mode == 1, cols_pad, p16);
        }
        FGX_CHECK_LAUNCH("fgx_pack_weight");
        return FGX_OK;
    }
    if (dtype == FGX_F32) pack_weight_kernel<float><<<grid, 256, 0, s>>>((const float*)weight, Ci, Co, V, mode, slab_bytes, slabs, cols_pad, (float*)panel);
    else pack_weight_kernel<uint16_t><<<grid, 256, 0, s>>>((const uint16_t*)weight, Ci, Co, V, mode, slab_bytes, slabs, cols_pad, (uint16_t*)panel);
    FGX_CHECK_LAUNCH("fgx_pack_weight");
    return FGX_OK;
}

size_t fgx_conv_scratch_bytes(size_t n, int cols, int splitk) {
    return splitk > 1 ? (size_t)splitk * n * (size_t)cols * sizeof(float) : 0;
}

int fgx_conv_gather_gemm(int dtype, const void* src, const void* panel, const void* bias, const uint32_t* map,
                         const int64_t* sorted_idx, const int32_t* tile_code, size_t n, int K, int cols, int V,
                         int tile_rows, int tile_cols, int slab_bytes, int splitk, void* scratch, void* out,
                         fgx_stream_t stream) {
    return fgx_conv_gather_gemm_act(dtype, src, panel, bias, map, sorted_idx, tile_code, n, K, cols, V, tile_rows, tile_cols,
                                    slab_bytes, splitk, scratch, FGX_ACT_NONE, out, stream);
}

int fgx_conv_gather_gemm_act(int dtype, const void* src, const void* panel, const void* bias, const uint32_t* map,
                             const int64_t* sorted_idx, const int32_t* tile_code, size_t n, int K, int cols, int V,
                             int tile_rows, int tile_cols, int slab_bytes, int splitk, void* scratch, int activation,
                             void* out, fgx_stream_t stream) {
    return fgx_conv_gather_gemm_act_mask(dtype, src, panel, bias, map, sorted_idx, tile_code, n, K, cols, V, tile_rows, tile_cols,
                                         slab_bytes, splitk, scratch, activation, out, nullptr, stream);
}

int fgx_conv_gather_gemm_act_mask(int dtype, const void* src, const void* panel, const void* bias, const uint32_t* map,
                                  const int64_t* sorted_idx, const int32_t* tile_code, size_t n, int K, int cols, int V,
                                  int tile_rows, int tile_cols, int slab_bytes, int splitk, void* scratch, int activation,
                                  void* out, uint8_t* relu_mask, fgx_stream_t stream) {
    FGX_CHECK_ARG(activation == FGX_ACT_NONE || activation == FGX_ACT_RELU, "fgx_conv_gather_gemm: unknown activation %d", activation);
    FGX_CHECK_ARG(relu_mask == nullptr || (activation == FGX_ACT_RELU && dtype != FGX_F32 && cols % 8 == 0),
                  "fgx_conv_gather_gemm: a ReLU mask needs the ReLU epilogue, a 16-bit type and a multiple of 8 columns (got %d)", cols);
    const int act = activation;
    FGX_CHECK_ARG(dtype_ok(dtype), "fgx_conv_gather_gemm: unknown dtype %d", dtype);
    FGX_CHECK_ARG(K > 0 && cols > 0 && V >= 1 && V <= 32, "fgx_conv_gather_gemm: bad shape K=%d cols=%d V=%d", K, cols, V);
    FGX_CHECK_ARG(splitk >= 1 && splitk <= 1024, "fgx_conv_gather_gemm: splitk %d out of range", splitk);
    FGX_CHECK_ARG(n < 0xFFFFFFFFull, "fgx_conv_gather_gemm: too many rows");
    if (n == 0) return FGX_OK;
    const int es = elem_size(dtype);
    FGX_CHECK_ARG(((size_t)K * es) % 16 == 0, "fgx_conv_gather_gemm: source row of %d elements is not a multiple of 16 bytes", K);
    FGX_CHECK_ARG(src && panel && map && sorted_idx && tile_code && out, "fgx_conv_gather_gemm: null buffer");
    FGX_CHECK_ARG((((uintptr_t)src | (uintptr_t)panel) & 15) == 0, "fgx_conv_gather_gemm: src and panel must be 16-byte aligned");
    FGX_CHECK_ARG(splitk == 1 || scratch != nullptr, "fgx_conv_gather_gemm: split-K needs a scratch buffer");
    FGX_CHECK_ARG(cdiv(n, tile_rows) <= 0x7FFFFFu, "fgx_conv_gather_gemm: too many row tiles");
    const int cols_pad = (int)align_up((size_t)cols, (size_t)tile_cols);
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case FGX_F16: return dispatch_tile<F16>(tile_rows, tile_cols, slab_bytes, src, panel, bias, map, sorted_idx, tile_code, n, K, cols, cols_pad, V, splitk, scratch, act, out, relu_mask, s);
        case FGX_BF16: return dispatch_tile<BF16>(tile_rows, tile_cols, slab_bytes, src, panel, bias, map, sorted_idx, tile_code, n, K, cols, cols_pad, V, splitk, scratch, act, out, relu_mask, s);
        default: return dispatch_tile<F32>(tile_rows, tile_cols, slab_bytes, src, panel, bias, map, sorted_idx, tile_code, n, K, cols, cols_pad, V, splitk, scratch, act, out, nullptr, s);
    }
}

int fgx_relu_mask_apply(int dtype, const void* grad, const uint8_t* relu_mask, size_t numel, void* out, fgx_stream_t stream) {
    FGX_CHECK_ARG(dtype == FGX_F16 || dtype == FGX_BF16, "fgx_relu_mask_apply: 16-bit types only (dtype %d)", dtype);
    FGX_CHECK_ARG(numel % 8 == 0, "fgx_relu_mask_apply: %zu elements are not a multiple of 8", numel);
    if (numel == 0) return FGX_OK;
    FGX_CHECK_ARG(grad && relu_mask && out, "fgx_relu_mask_apply: null buffer");
    FGX_CHECK_ARG((((uintptr_t)grad | (uintptr_t)out) & 15) == 0, "fgx_relu_mask_apply: grad and out must be 16-byte aligned");
    const size_t pieces = numel / 8;
    unsigned grid = cdiv(pieces, 256);
    if (grid > 16384u) grid = 16384u;
    relu_mask_apply_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const u32x4*)grad, relu_mask, pieces, (u32x4*)out);
    FGX_CHECK_LAUNCH("fgx_relu_mask_apply");
    return FGX_OK;
}

size_t fgx_colsum_scratch_bytes(size_t n, int cols) {
    (void)n;
    return (size_t)kColsumSlices * (size_t)(cols > 0 ? cols : 1) * sizeof(float);
}

int fgx_colsum(int dtype, const void* x, size_t n, int cols, void* scratch, void* out, fgx_stream_t stream) {
    FGX_CHECK_ARG(dtype_ok(dtype), "fgx_colsum: unknown dtype %d", dtype);
    FGX_CHECK_ARG(cols > 0 && out != nullptr, "fgx_colsum: bad shape or null output");
    FGX_CHECK_ARG(scratch != nullptr && (n == 0 || x != nullptr), "fgx_colsum: null buffer");
    return colsum_launch(dtype, x, n, cols, (float*)scratch, out, (hipStream_t)stream);
}

int fgx_colsum_static_max_cols(void) { return kStaticColsumCols; }

// The device address of the current GPU's copy of the scratch array, looked up once per device with that device current.
// The lookup may load the code object and is no stream operation: it must not happen while a stream is being captured.
static int static_colsum_ptr(const char* who, hipStream_t s, float** out) {
    int dev = 0;
    FGX_CHECK_HIP(hipGetDevice(&dev));
    FGX_CHECK_ARG(dev >= 0 && dev < kMaxDevices, "%s: device ordinal %d out of range", who, dev);
    float* ptr = g_static_colsum_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &capturing) == hipSuccess && capturing != hipStreamCaptureStatusNone) {
            (void)hipGetLastError();
            set_error("%s: first use on device %d while its stream is being captured; call fgx_colsum_static_prepare() on this device before the capture", who, dev);
            return FGX_ERR_ARG;
        }
        void* found = nullptr;
        FGX_CHECK_HIP(hipGetSymbolAddress(&found, HIP_SYMBOL(g_static_colsum_scratch)));
        FGX_CHECK_ARG(found != nullptr, "%s: the scratch array has no address on device %d", who, dev);
        ptr = (float*)found;
        g_static_colsum_ptr[dev].store(ptr, std::memory_order_release);     // (two first callers find the same address)
    }
    *out = ptr;
    return FGX_OK;
}

int fgx_colsum_static_prepare(void) {
    float* ptr = nullptr;
    return static_colsum_ptr("fgx_colsum_static_prepare", nullptr, &ptr);
}

int fgx_colsum_static(int dtype, const void* x, size_t n, int cols, void* out, fgx_stream_t stream) {
    FGX_CHECK_ARG(dtype_ok(dtype), "fgx_colsum_static: unknown dtype %d", dtype);
    FGX_CHECK_ARG(cols > 0 && out != nullptr, "fgx_colsum_static: bad shape or null output");
    FGX_CHECK_ARG(n == 0 || x != nullptr, "fgx_colsum_static: null buffer");
    FGX_CHECK_ARG(cols <= kStaticColsumCols,
                  "fgx_colsum_static: %d columns exceed the %d the library's own scratch holds; use fgx_colsum with caller-owned scratch",
                  cols, kStaticColsumCols);
    float* ptr = nullptr;
    const int rc = static_colsum_ptr("fgx_colsum_static", (hipStream_t)stream, &ptr);
    if (rc != FGX_OK) return rc;
    return colsum_launch(dtype, x, n, cols, ptr, out, (hipStream_t)stream);
}

}  // extern "C"
