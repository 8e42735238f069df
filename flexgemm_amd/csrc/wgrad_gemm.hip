// Weight gradient of the submanifold sparse conv on gfx950: a pair-list GEMM per kernel offset.
//
//   grad_weight[co, v, ci] = sum over pairs k of offset v of grad_out[sig_o[k], co] * feats[sig_i[k], ci]
//
// The contraction runs over pairs, i.e. over ROWS of both operands, while MFMA fragments want the
// contraction index contiguous inside a lane.  Rows are staged in LDS pair-major, exactly as they sit in
// memory; 16-bit fragments are then read with the gfx950 transposing LDS load (ds_read_b64_tr_b16: a
// 16-lane group reads a 4-pair x 16-channel block and each lane receives the 4 pair values of its own
// channel), fp32 fragments with plain 32-bit reads.
//
// Pipeline.  Both operands are gathers, and each gather depends on an index (sig_o / sig_i) that has to
// be fetched first.  Everything moves with direct global->LDS loads (lane i of a wavefront deposits its
// data at LDS base + size * i) through two rings: an index ring (32 + 32 indices per step) that runs
// 2 (S-1) steps ahead, and a row ring of S stages (32 pair rows of each operand) that runs S-1 steps ahead
// and takes its addresses from the index ring.  These loads are the only vector-memory operations in the
// main loop and every wavefront issues the same number per step (dummy loads past the end), so
// s_waitcnt vmcnt((S-2) * loads_per_step) means "this step's rows and the indices needed for the next
// enqueue have landed"; one workgroup barrier per step publishes them.
//
// Work decomposition and locality.  Inside one offset's segment the pairs are ordered by output row,
// and the matching input rows are that row's neighbors, so the pairs of ALL offsets that belong to one
// block of `block_rows` consecutive voxels touch the same few megabytes of grad_out / feats.  A work item
// is therefore (voxel block b, offset v, Co-tile, Ci-tile); the item list is block-major and each XCD takes
// a contiguous eighth of it (workgroup ids are dealt round-robin over the 8 XCDs), so the items of one voxel
// block run back to back on one XCD: the rows are fetched from HBM once and then served by that XCD's L2 to
// the other offsets.  Each item writes an
// fp32 partial product; a second kernel adds an offset's partials in block order (deterministic) and
// casts to the output type.  The per-(offset, block) pair ranges are found by a small binary-search
// kernel over sig_o.
#include <type_traits>

#include "wgrad_device.h"

namespace fgx {
namespace {

constexpr int kStages = 4;      // row ring depth
constexpr int kIdxSlots = 8;    // index ring depth (>= kStages, power of two)

// 16 zero bytes every lane may read: pairs past the end of an item, columns past the tensor width
__device__ __attribute__((aligned(256))) unsigned char g_zero_block_w[256];

template <typename Tag, int BM, int BN, int WAVES_M, int WAVES_N>
struct WgradCfg {
    using T = typename Tag::type;
    static constexpr int ES = (int)sizeof(T);
    static constexpr int NW = WAVES_M * WAVES_N;
    static constexpr int NT = 64 * NW;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int TM = WM / 32, TN = WN / 32;
    static constexpr int PAIRS = 32;                                   // pairs per pipeline step
    static constexpr int ROWB_A = BM * ES, ROWB_B = BN * ES;           // bytes of one staged pair row
    static constexpr int CH_A = ROWB_A / 16, CH_B = ROWB_B / 16;       // 16-byte chunks per row
    static constexpr int RPI_A = 64 / CH_A, RPI_B = 64 / CH_B;         // pair rows one wave-wide load covers
    static constexpr int A_INST = PAIRS / RPI_A, B_INST = PAIRS / RPI_B;
    static constexpr int A_PER = (A_INST + NW - 1) / NW, B_PER = (B_INST + NW - 1) / NW;
    static constexpr int LPS = A_PER + B_PER + 1;                      // + one index load
    static constexpr int A_BYTES = PAIRS * ROWB_A, B_BYTES = PAIRS * ROWB_B;
    static constexpr int STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int IDX_SLOT_BYTES = 64 * 4;                      // 32 sig_o + 32 sig_i
    static constexpr size_t lds_bytes = (size_t)kStages * STAGE_BYTES + (size_t)kIdxSlots * IDX_SLOT_BYTES + 1024;
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert(CH_A <= 64 && CH_B <= 64 && 64 % CH_A == 0 && 64 % CH_B == 0, "row slice must divide a wave-wide load");
    static_assert((kStages - 2) * LPS < 64, "outstanding loads exceed the vmcnt range");
    // XOR key on the 16-byte chunk index: the transposing read touches 4 consecutive pair rows x 32 bytes, which
    // must fall into distinct bank groups
    static constexpr int key_a(int row) { return ES != 2 ? 0 : (CH_A >= 16 ? 4 * (row & 3) : (CH_A >= 8 ? 2 * (row & 3) : 0)); }
    static constexpr int key_b(int row) { return ES != 2 ? 0 : (CH_B >= 16 ? 4 * (row & 3) : (CH_B >= 8 ? 2 * (row & 3) : 0)); }
};

template <typename Tag, int BM, int BN, int WAVES_M, int WAVES_N>
__global__ void __launch_bounds__(64 * WAVES_M * WAVES_N)
wgrad_kernel(const typename Tag::type* __restrict__ gout, const typename Tag::type* __restrict__ feats,
             const uint32_t* __restrict__ sig_i, const uint32_t* __restrict__ sig_o,
             const uint32_t* __restrict__ bounds, int V, int Ci, int Co, unsigned nb, unsigned co_tiles,
             unsigned ci_tiles, bool small_tensors, float* __restrict__ partial,
             typename Tag::type* __restrict__ direct) {
    using C = WgradCfg<Tag, BM, BN, WAVES_M, WAVES_N>;
    constexpr int ES = C::ES;
    constexpr int S = kStages;

    // XCD-aware item order.  Items are listed block-major (block, offset, tile); workgroup ids are dealt round-robin
    // over the 8 XCDs, so XCD x takes the x-th contiguous eighth of the list: the items of one voxel block run on one
    // XCD back to back (or on a few neighbouring XCDs when there are fewer blocks than XCDs).
    const unsigned tiles = co_tiles * ci_tiles;
    const unsigned per_block = (unsigned)V * tiles;
    const unsigned total_items = nb * per_block;
    const unsigned per_xcd = (total_items + kXcds - 1) / kXcds;
    const unsigned item = (blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
    if (blockIdx.x / kXcds >= per_xcd || item >= total_items) return;
    const unsigned b = item / per_block;
    const unsigned within = item % per_block;
    const unsigned v = within / tiles;
    const unsigned tile = within % tiles;
    const unsigned co_tile = tile % co_tiles, ci_tile = tile / co_tiles;
    const uint32_t k_lo = bounds[v * (nb + 1) + b];
    const uint32_t k_hi = bounds[v * (nb + 1) + b + 1];
    if (k_lo >= k_hi) return;   // the reduction skips empty items
    const int nsteps = (int)((k_hi - k_lo + C::PAIRS - 1) / C::PAIRS);

    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    unsigned char* ring = lds_raw;                                              // [S][A rows | B rows]
    unsigned char* idx_ring = ring + S * C::STAGE_BYTES;                        // [kIdxSlots][o x 32 | i x 32]
    unsigned char* dump = idx_ring + kIdxSlots * C::IDX_SLOT_BYTES;             // sink of surplus loads

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const int g = lane >> 5, l32 = lane & 31;
    const int m0 = (int)co_tile * BM, n0 = (int)ci_tile * BN;
    const unsigned char* gout_b = (const unsigned char*)gout;
    const unsigned char* feats_b = (const unsigned char*)feats;
    const unsigned char* zero_b = g_zero_block_w;
    const size_t rowb_o = (size_t)Co * ES, rowb_i = (size_t)Ci * ES;

    f32x16 acc[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    // index slot of step j: lanes 0-31 fetch sig_o, lanes 32-63 sig_i of the step's 32 pairs and deposit them at
    // slot + 4 * lane.  Every wavefront issues the same load (same data, same place) so that all of them count alike.
    auto issue_idx = [&](int j) {
        uint32_t k = k_lo + (uint32_t)j * C::PAIRS + (uint32_t)(lane & 31);
        k = k < k_hi ? k : k_hi - 1;                       // past the end: any valid address, the row load ignores it
        const uint32_t* src = (lane & 32) ? sig_i + k : sig_o + k;
        unsigned char* dst = idx_ring + (j & (kIdxSlots - 1)) * C::IDX_SLOT_BYTES;
        __builtin_amdgcn_global_load_lds(FGX_GLOBAL_PTR(src), FGX_LDS_PTR(dst), 4, 0, 0);
    };
    // rows of step j into stage j % S; exactly A_PER + B_PER loads per wavefront.  Steps whose 32 pairs all exist,
    // in tiles that lie fully inside tensors of less than 4 GiB, take a lean path (32-bit offsets from a uniform base,
    // no validity selects); the last partial step, edge tiles, huge tensors and the dummy steps take the general one.
    int a_row[C::A_PER], a_colb[C::A_PER], b_row[C::B_PER], b_colb[C::B_PER];
    bool a_mine[C::A_PER], b_mine[C::B_PER];
#pragma unroll
    for (int i = 0; i < C::A_PER; ++i) {
        const int inst = i * C::NW + wave;
        a_mine[i] = C::A_INST % C::NW == 0 || inst < C::A_INST;               // wave-uniform
        a_row[i] = (a_mine[i] ? inst : 0) * C::RPI_A + lane / C::CH_A;
        a_colb[i] = (m0 + ((lane % C::CH_A) ^ C::key_a(a_row[i])) * (16 / ES)) * ES;   // byte column in the tensor row
    }
#pragma unroll
    for (int i = 0; i < C::B_PER; ++i) {
        const int inst = i * C::NW + wave;
        b_mine[i] = C::B_INST % C::NW == 0 || inst < C::B_INST;               // wave-uniform
        b_row[i] = (b_mine[i] ? inst : 0) * C::RPI_B + lane / C::CH_B;
        b_colb[i] = (n0 + ((lane % C::CH_B) ^ C::key_b(b_row[i])) * (16 / ES)) * ES;
    }
    const int full_steps = (int)((k_hi - k_lo) / C::PAIRS);
    const bool lean_ok = m0 + BM <= Co && n0 + BN <= Ci && small_tensors &&
                         C::A_INST % C::NW == 0 && C::B_INST % C::NW == 0;      // uniform
    auto issue_rows = [&](int j) {
        unsigned char* stage = ring + (j & (S - 1)) * C::STAGE_BYTES;
        const uint32_t* slot_p = (const uint32_t*)(idx_ring + (j & (kIdxSlots - 1)) * C::IDX_SLOT_BYTES);
        if (lean_ok && j < full_steps) {
            uint32_t oa[C::A_PER], ob[C::B_PER];
#pragma unroll
            for (int i = 0; i < C::A_PER; ++i) oa[i] = slot_p[a_row[i]] * (uint32_t)rowb_o + (uint32_t)a_colb[i];
#pragma unroll
            for (int i = 0; i < C::B_PER; ++i) ob[i] = slot_p[32 + b_row[i]] * (uint32_t)rowb_i + (uint32_t)b_colb[i];
#pragma unroll
            for (int i = 0; i < C::A_PER; ++i)
                __builtin_amdgcn_global_load_lds(FGX_GLOBAL_PTR(gout_b + oa[i]), FGX_LDS_PTR(stage + (i * C::NW + wave) * 1024), 16, 0, 0);
#pragma unroll
            for (int i = 0; i < C::B_PER; ++i)
                __builtin_amdgcn_global_load_lds(FGX_GLOBAL_PTR(feats_b + ob[i]), FGX_LDS_PTR(stage + C::A_BYTES + (i * C::NW + wave) * 1024), 16, 0, 0);
            return;
        }
        const bool live = j < nsteps;
        const uint32_t kbase = k_lo + (uint32_t)j * C::PAIRS;
#pragma unroll
        for (int i = 0; i < C::A_PER; ++i) {
            const uint32_t o = slot_p[a_row[i]];
            const bool real = live && a_mine[i] && kbase + (uint32_t)a_row[i] < k_hi && a_colb[i] < Co * ES;
            const size_t off = real ? (size_t)o * rowb_o + (size_t)a_colb[i] : (size_t)0;
            const unsigned char* p = real ? gout_b + off : zero_b;
            unsigned char* dst = a_mine[i] ? stage + (i * C::NW + wave) * 1024 : dump;
            __builtin_amdgcn_global_load_lds(FGX_GLOBAL_PTR(p), FGX_LDS_PTR(dst), 16, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < C::B_PER; ++i) {
            const uint32_t ii = slot_p[32 + b_row[i]];
            const bool real = live && b_mine[i] && kbase + (uint32_t)b_row[i] < k_hi && b_colb[i] < Ci * ES;
            const size_t off = real ? (size_t)ii * rowb_i + (size_t)b_colb[i] : (size_t)0;
            const unsigned char* p = real ? feats_b + off : zero_b;
            unsigned char* dst = b_mine[i] ? stage + C::A_BYTES + (i * C::NW + wave) * 1024 : dump;
            __builtin_amdgcn_global_load_lds(FGX_GLOBAL_PTR(p), FGX_LDS_PTR(dst), 16, 0, 0);
        }
    };

    // ---- prologue: indices of the first S-1 steps, then S-1 enqueue rounds ----
#pragma unroll
    for (int j = 0; j < S - 1; ++j) issue_idx(j);
    wait_vmcnt<0>();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll
    for (int j = 0; j < S - 1; ++j) {
        issue_rows(j);
        issue_idx(j + S - 1);
    }

    // fragment addressing (constant per lane)
    const int s16 = lane & 15, mb = (lane >> 4) & 1;
    for (int k = 0; k < nsteps; ++k) {
        wait_vmcnt<(S - 2) * C::LPS>();    // rows of step k and the indices of step k+S-1 have landed
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        issue_rows(k + S - 1);
        issue_idx(k + 2 * (S - 1));
        const unsigned char* a_cur = ring + (k & (S - 1)) * C::STAGE_BYTES;
        const unsigned char* b_cur = a_cur + C::A_BYTES;
        if constexpr (ES == 2) {
            // Transposing read: in a 16-lane group, lane s supplies the address of 4 adjacent channels of pair
            // row (s / 4) and receives the 4 pair values of channel (group base + s).  Lanes 0-15 / 16-31 cover
            // fragment rows 0-15 / 16-31, the two wave halves take pair rows [0, 8) / [8, 16) of the k-step.
            constexpr int NK = C::PAIRS / 16;
            i16x4 ar[NK * C::TM * 2], br[NK * C::TN * 2];      // (lo, hi) halves of every fragment of the step
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) {
                const int prow = kk * 16 + g * 8 + (s16 >> 2);
#pragma unroll
                for (int i = 0; i < C::TM; ++i) {
                    const int byte = (wave_m * C::WM + i * 32 + mb * 16 + (s16 & 3) * 4) * 2;
                    const int c = byte >> 4, w = byte & 15;
                    ar[(kk * C::TM + i) * 2] = lds_read_tr16(a_cur + prow * C::ROWB_A + ((c ^ C::key_a(prow)) << 4) + w);
                    ar[(kk * C::TM + i) * 2 + 1] = lds_read_tr16(a_cur + (prow + 4) * C::ROWB_A + ((c ^ C::key_a(prow + 4)) << 4) + w);
                }
#pragma unroll
                for (int j = 0; j < C::TN; ++j) {
                    const int byte = (wave_n * C::WN + j * 32 + mb * 16 + (s16 & 3) * 4) * 2;
                    const int c = byte >> 4, w = byte & 15;
                    br[(kk * C::TN + j) * 2] = lds_read_tr16(b_cur + prow * C::ROWB_B + ((c ^ C::key_b(prow)) << 4) + w);
                    br[(kk * C::TN + j) * 2 + 1] = lds_read_tr16(b_cur + (prow + 4) * C::ROWB_B + ((c ^ C::key_b(prow + 4)) << 4) + w);
                }
            }
            lds_wait_all(ar);
            lds_wait_all(br);
#pragma unroll
            for (int kk = 0; kk < NK; ++kk)
#pragma unroll
                for (int i = 0; i < C::TM; ++i)
#pragma unroll
                    for (int j = 0; j < C::TN; ++j) {
                        const i16x8 af = __builtin_shufflevector(ar[(kk * C::TM + i) * 2], ar[(kk * C::TM + i) * 2 + 1], 0, 1, 2, 3, 4, 5, 6, 7);
                        const i16x8 bf = __builtin_shufflevector(br[(kk * C::TN + j) * 2], br[(kk * C::TN + j) * 2 + 1], 0, 1, 2, 3, 4, 5, 6, 7);
                        mma16<Tag>(acc[i][j], af, bf);
                    }
        } else {
            // fp32: one value per lane and MFMA (32x32x2); lane group g takes the odd / even pair of each couple
#pragma unroll
            for (int kk = 0; kk < C::PAIRS / 2; ++kk) {
                const int p = kk * 2 + g;
                float af[C::TM], bf[C::TN];
#pragma unroll
                for (int i = 0; i < C::TM; ++i) af[i] = *(const float*)(a_cur + p * C::ROWB_A + (wave_m * C::WM + i * 32 + l32) * 4);
#pragma unroll
                for (int j = 0; j < C::TN; ++j) bf[j] = *(const float*)(b_cur + p * C::ROWB_B + (wave_n * C::WN + j * 32 + l32) * 4);
#pragma unroll
                for (int i = 0; i < C::TM; ++i)
#pragma unroll
                    for (int j = 0; j < C::TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
            }
        }
    }
    wait_vmcnt<0>();   // the trailing dummy loads

    // partial[b][v][co][ci], fp32 -- or, when there is a single voxel block, straight into grad_weight[co][v][ci]
    float* dst = partial + ((size_t)b * V + v) * ((size_t)Co * Ci);
    typename Tag::type* out = direct ? direct + (size_t)v * Ci : nullptr;
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
        const int ci = n0 + wave_n * C::WN + j * 32 + l32;
        if (ci >= Ci) continue;
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                int co = m0 + wave_m * C::WM + i * 32 + (e >> 2) * 8 + g * 4 + (e & 3);
                if (co < Co) {
                    if (out) out[(size_t)co * V * Ci + ci] = from_float<typename Tag::type>(acc[i][j][e]);
                    else dst[(size_t)co * Ci + ci] = acc[i][j][e];
                }
            }
    }
}

// ------------------------------------------------------------------------------------------------
// Streaming variant (16-bit types): one persistent workgroup per CU, specialised wavefronts.
// ------------------------------------------------------------------------------------------------
// Four wavefronts multiply (2 x 2 over the Co x Ci tile), four more only enqueue loads: issuing a vector-memory
// instruction blocks its wavefront while the address pipeline is busy, and a step's gathers keep that pipeline busy
// for longer than its MFMAs take, so the two kinds of work sit in different wavefronts.  A workgroup walks its share
// of the block-major item list (XCD x takes the x-th eighth, its workgroups interleave inside it) and treats the
// 64-pair steps of all its items as one stream through a 4-stage row ring and an 8-slot index ring, so the loads of
// the next item are in flight while the current one finishes.  Loads are buffer loads into LDS: a pair past the end
// of an item or a column past the tensor is an out-of-range offset and arrives as zeros.  A loader's outstanding-
// load counter sees only its own loads in issue order: "step c has landed" is s_waitcnt vmcnt(loads issued in the
// last two iterations).
constexpr int kWsStages = 4;
constexpr int kWsIdxSlots = 8;
constexpr int kWsIdxAhead = 4;       // index loads run this many steps ahead of the row loads (> kWsStages - 1)
constexpr int kWsLoaders = 4;
constexpr int kWsPairs = 64;         // pairs per step
template <typename Tag, int BM, int BN>
struct WStreamCfg {
    using T = typename Tag::type;
    static constexpr int ES = (int)sizeof(T);
    // A 32 x 32 tile is one MFMA tile: the four multipliers then split the PAIRS of a step among themselves (each owns a
    // quarter of the pair rows and keeps its own accumulator, written out as a partial product of its own), and a step
    // carries four times the pairs so that its loads are as many bytes as a wide tile's.
    static constexpr bool KSPLIT = BM == 32 && BN == 32;
    static constexpr int SLICES = KSPLIT ? 4 : 1;                  // partial products per (voxel block, offset, tile)
    // (a 256 x 128 tile's stages are 48 KiB: three of them fit, with the same 64-pair steps)
    static constexpr int P = KSPLIT ? 4 * kWsPairs : kWsPairs, S = BM * BN > 128 * 128 ? 3 : kWsStages;
    static constexpr int NW = 4, NL = kWsLoaders, NT = 64 * (NW + NL);
    static constexpr int WM = KSPLIT ? BM : BM / 2, WN = KSPLIT ? BN : BN / 2, TM = WM / 32, TN = WN / 32;
    static constexpr int IDX_PER = P / 64;                         // wave-wide index loads per operand and step
    static constexpr int ROWB_A = BM * ES, ROWB_B = BN * ES;
    static constexpr int CH_A = ROWB_A / 16, CH_B = ROWB_B / 16;
    static constexpr int RPI_A = 64 / CH_A, RPI_B = 64 / CH_B;
    static constexpr int A_PER = P / RPI_A / NL, B_PER = P / RPI_B / NL;
    static constexpr int LPS = A_PER + B_PER;
    static constexpr int A_BYTES = P * ROWB_A, B_BYTES = P * ROWB_B, STAGE_BYTES = A_BYTES + B_BYTES;
    static constexpr int IDX_SLOT_BYTES = 2 * P * 4;               // sig_o x P | sig_i x P
    static constexpr size_t lds_bytes = (size_t)S * STAGE_BYTES + (size_t)kWsIdxSlots * IDX_SLOT_BYTES;
    static_assert(ES == 2, "the streaming kernel handles 16-bit types");
    static_assert(S == 3 || S == 4, "the loaders' wait is written for rings of three or four stages");
    static_assert(kWsIdxAhead > S - 1 && lds_bytes <= 160 * 1024, "index loads run ahead of the row loads; the ring fits LDS");
    static_assert(IDX_PER == 1 || IDX_PER == NL, "index loads: one loader per operand, or every loader a quarter of both");
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of 32x32");
    static_assert(P % (RPI_A * NL) == 0 && P % (RPI_B * NL) == 0, "every loader issues the same row loads");
    static_assert(2 * (LPS + 1) < 64, "outstanding loads exceed the vmcnt range");
    static constexpr int key_a(int row) { return CH_A >= 16 ? 4 * (row & 3) : (CH_A >= 8 ? 2 * (row & 3) : 0); }
    static constexpr int key_b(int row) { return CH_B >= 16 ? 4 * (row & 3) : (CH_B >= 8 ? 2 * (row & 3) : 0); }
};

template <typename Tag, int BM, int BN>
__global__ void __launch_bounds__(64 * (4 + kWsLoaders))
wgrad_stream_kernel(const typename Tag::type* __restrict__ gout, const typename Tag::type* __restrict__ feats,
                    const uint32_t* __restrict__ sig_i, const uint32_t* __restrict__ sig_o,
                    const uint32_t* __restrict__ bounds, int V, int Ci, int Co, unsigned nb, unsigned co_tiles,
                    unsigned ci_tiles, uint32_t n_pairs, uint32_t gout_bytes, uint32_t feats_bytes,
                    float* __restrict__ partial, typename Tag::type* __restrict__ direct,
                    float* __restrict__ bias_partial, int bias_offset, const uint32_t* __restrict__ lists) {
    using C = WStreamCfg<Tag, BM, BN>;
    constexpr int ES = C::ES, S = C::S, P = C::P;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    unsigned char* ring = lds_raw;                                              // [S][A rows | B rows]
    uint32_t* idx_ring = (uint32_t*)(ring + S * C::STAGE_BYTES);                // [kWsIdxSlots][o x P | i x P]

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool loader = wave >= C::NW;
    const int lw = loader ? wave - C::NW : 0, mw = loader ? 0 : wave;
    const int wave_m = C::KSPLIT ? 0 : mw >> 1, wave_n = C::KSPLIT ? 0 : mw & 1;
    const int g = lane >> 5, l32 = lane & 31;

    // ---- item list: block-major (block, offset, tile); XCD x owns the x-th eighth, its workgroups interleave ----
    // With `lists` (head[workgroups] | next[items], kItemListEnd closes a chain) a workgroup walks the chain that the
    // balancing pass made for it instead.
    const unsigned tiles = co_tiles * ci_tiles;
    const unsigned per_block = (unsigned)V * tiles;
    const unsigned total_items = nb * per_block;
    const unsigned per_xcd = (total_items + kXcds - 1) / kXcds;
    const unsigned xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds, stride = gridDim.x / kXcds;
    // (lists made for another launch shape are ignored: every partition of the items gives the same result, a list of
    // the wrong size does not)
    if (lists && !(lists[0] == gridDim.x && lists[1] == total_items && lists[2] == tiles && lists[3] == kItemListMagic)) lists = nullptr;
    if (lists) lists += kItemListHeader;
    const unsigned range_end = lists ? total_items : ((xcd + 1) * per_xcd < total_items ? (xcd + 1) * per_xcd : total_items);
    const uint32_t* chain = lists ? lists + gridDim.x : nullptr;
    auto after = [&](unsigned item) -> unsigned { return chain ? chain[item] : item + stride; };

    struct Walk {
        unsigned item;
        uint32_t k, k_hi;       // next pair to hand out, end of the item's pairs
        unsigned b, v, tile;
        bool live;
    };
    auto seek = [&](Walk& w) {                      // settle on the first non-empty item at or after w.item
        w.live = false;
        while (w.item < range_end) {
            const unsigned b = w.item / per_block, within = w.item % per_block;
            const unsigned v = within / tiles;
            const uint32_t lo = bounds[v * (nb + 1) + b], hi = bounds[v * (nb + 1) + b + 1];
            if (lo < hi) {
                w.k = lo;
                w.k_hi = hi;
                w.b = b;
                w.v = v;
                w.tile = within % tiles;
                w.live = true;
                return;
            }
            w.item = after(w.item);
        }
    };
    auto advance = [&](Walk& w) {                   // one step further
        w.k += P;
        if (w.k >= w.k_hi) {
            w.item = after(w.item);
            seek(w);
        }
    };
    Walk first;
    first.item = lists ? lists[blockIdx.x] : xcd * per_xcd + slot;
    seek(first);
    if (!first.live) return;                        // whole workgroup: nothing to do

    const rsrc_t gout_rs = make_rsrc(gout, gout_bytes);
    const rsrc_t feats_rs = make_rsrc(feats, feats_bytes);
    const rsrc_t sigo_rs = make_rsrc(sig_o, n_pairs * 4u);
    const rsrc_t sigi_rs = make_rsrc(sig_i, n_pairs * 4u);
    const uint32_t rowb_o = (uint32_t)Co * ES, rowb_i = (uint32_t)Ci * ES;

    if (loader) {
        // =============================================================================================
        // loaders
        // =============================================================================================
        int a_row[C::A_PER], b_row[C::B_PER];
        uint32_t a_chb[C::A_PER], b_chb[C::B_PER];          // byte column inside the tile, swizzle applied
#pragma unroll
        for (int i = 0; i < C::A_PER; ++i) {
            a_row[i] = (i * C::NL + lw) * C::RPI_A + lane / C::CH_A;
            a_chb[i] = (uint32_t)(((lane % C::CH_A) ^ C::key_a(a_row[i])) * 16);
        }
#pragma unroll
        for (int i = 0; i < C::B_PER; ++i) {
            b_row[i] = (i * C::NL + lw) * C::RPI_B + lane / C::CH_B;
            b_chb[i] = (uint32_t)(((lane % C::CH_B) ^ C::key_b(b_row[i])) * 16);
        }
        Walk f = first, r = first;                  // index stream, row stream
        unsigned f_step = 0, r_step = 0;            // steps handed out so far (ring positions)
        auto issue_idx = [&]() -> int {             // index loads of the index stream's next step
            if (!f.live) return 0;
            int ops = 0;
            uint32_t* dst = idx_ring + (f_step & (kWsIdxSlots - 1)) * (2 * P);
            if constexpr (C::IDX_PER == 1) {
                if (lw == 0) {
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(sigo_rs, FGX_LDS_PTR(dst), 4, (f.k + (uint32_t)lane) * 4u, 0, 0, 0);
                    ops = 1;
                } else if (lw == 1) {
                    uint32_t* dst_i = dst + P;
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(sigi_rs, FGX_LDS_PTR(dst_i), 4, (f.k + (uint32_t)lane) * 4u, 0, 0, 0);
                    ops = 1;
                }
            } else {        // every loader fetches its quarter of both index columns
                const uint32_t vo = (f.k + (uint32_t)(lw * 64 + lane)) * 4u;
                uint32_t* dst_o = dst + lw * 64;
                uint32_t* dst_i = dst + P + lw * 64;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(sigo_rs, FGX_LDS_PTR(dst_o), 4, vo, 0, 0, 0);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(sigi_rs, FGX_LDS_PTR(dst_i), 4, vo, 0, 0, 0);
                ops = 2;
            }
            ++f_step;
            advance(f);
            return ops;
        };
        // Row loads come in two halves.  prep_rows() turns the next step's indices into per-lane buffer offsets (LDS
        // reads, multiplies, range checks) and is run right AFTER the previous step's loads were enqueued, i.e. while the
        // multipliers work and this wavefront would only wait for the next barrier; fire_rows() then enqueues the
        // prepared loads first thing after that barrier.
        bool pr_live = false;
        unsigned pr_stage = 0;
        uint32_t va[C::A_PER], vb[C::B_PER];
        auto prep_rows = [&]() {
            pr_live = r.live;
            if (!r.live) return;
            pr_stage = r_step % S;
            const uint32_t* slot_p = idx_ring + (r_step & (kWsIdxSlots - 1)) * (2 * P);
            const unsigned co_tile = r.tile % co_tiles, ci_tile = r.tile / co_tiles;
            const uint32_t m0b = co_tile * (uint32_t)(BM * ES), n0b = ci_tile * (uint32_t)(BN * ES);
            const uint32_t left = r.k_hi - r.k;                                   // pairs left in the item
            const bool ragged = left < (uint32_t)P || m0b + BM * ES > rowb_o || n0b + BN * ES > rowb_i;   // uniform
#pragma unroll
            for (int i = 0; i < C::A_PER; ++i) va[i] = slot_p[a_row[i]] * rowb_o + (m0b + a_chb[i]);
#pragma unroll
            for (int i = 0; i < C::B_PER; ++i) vb[i] = slot_p[P + b_row[i]] * rowb_i + (n0b + b_chb[i]);
            if (ragged) {
#pragma unroll
                for (int i = 0; i < C::A_PER; ++i)
                    va[i] = ((uint32_t)a_row[i] < left && m0b + a_chb[i] < rowb_o) ? va[i] : kOobOffset;
#pragma unroll
                for (int i = 0; i < C::B_PER; ++i)
                    vb[i] = ((uint32_t)b_row[i] < left && n0b + b_chb[i] < rowb_i) ? vb[i] : kOobOffset;
            }
            ++r_step;
            advance(r);
        };
        auto fire_rows = [&]() -> int {             // 0 when the stream is over
            if (!pr_live) return 0;
            unsigned char* stage = ring + pr_stage * C::STAGE_BYTES;
            // (offsets go through a scalar local: the host pass of hipcc silently drops a kernel whose body hands an
            // array element straight to this builtin)
#pragma unroll
            for (int i = 0; i < C::A_PER; ++i) {
                const uint32_t vo = va[i];
                __builtin_amdgcn_raw_ptr_buffer_load_lds(gout_rs, FGX_LDS_PTR(stage + (i * C::NL + lw) * 1024), 16, vo, 0, 0, 0);
            }
            unsigned char* stage_b = stage + C::A_BYTES;
#pragma unroll
            for (int i = 0; i < C::B_PER; ++i) {
                const uint32_t vo = vb[i];
                __builtin_amdgcn_raw_ptr_buffer_load_lds(feats_rs, FGX_LDS_PTR(stage_b + (i * C::NL + lw) * 1024), 16, vo, 0, 0, 0);
            }
            return C::LPS;
        };
        // at most `n` of this loader's loads may be outstanding; n is a sum of two per-iteration counts, each 0, LPS
        // or LPS + 1 (rounded down to the next value handled here, which is merely stricter)
        auto wait_loads = [&](int n) {
            if (n >= 2 * C::LPS + 2) wait_vmcnt<2 * C::LPS + 2>();
            else if (n == 2 * C::LPS + 1) wait_vmcnt<2 * C::LPS + 1>();
            else if (n == 2 * C::LPS) wait_vmcnt<2 * C::LPS>();
            else if (n > C::LPS) wait_vmcnt<C::LPS + 1>();
            else if (n == C::LPS) wait_vmcnt<C::LPS>();
            else wait_vmcnt<0>();
        };

        // prologue: indices of the first kWsIdxAhead steps, then S-1 row rounds
#pragma unroll
        for (int j = 0; j < kWsIdxAhead; ++j) (void)issue_idx();
        wait_vmcnt<0>();
        __syncthreads();
        prep_rows();
        int drained = 0, ops1 = 0, ops2 = 0;        // ops1: loads issued in the previous round, ops2: the one before
#pragma unroll
        for (int j = 0; j < S - 1; ++j) {
            int ops = fire_rows();
            if (ops == 0) ++drained;
            prep_rows();                            // indices of steps 1 .. S-1 came with the first batch
            ops += issue_idx();
            ops2 = ops1;
            ops1 = ops;
        }
        while (true) {
            // everything issued before the last S - 2 rounds has landed: the rows of the step the barrier opens
            wait_loads(S == 4 ? ops1 + ops2 : ops1);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();          // ... everybody's; the stage multiplied in the previous step is free
            asm volatile("" ::: "memory");
            int ops = fire_rows();
            if (ops == 0) ++drained;
            if (drained >= S - 1) break;           // that was the barrier of the stream's last step
            prep_rows();
            ops += issue_idx();
            ops2 = ops1;
            ops1 = ops;
        }
        wait_vmcnt<0>();
        return;
    }

    // =================================================================================================
    // multipliers
    // =================================================================================================
    __syncthreads();                                // the loaders' prologue barrier
    const int s16 = lane & 15, mb = (lane >> 4) & 1;
    constexpr int NK = P / 16 / C::SLICES;          // k-blocks (16 pair rows) this wavefront multiplies per step
    const int kk0 = C::KSPLIT ? mw * NK : 0;        // ... starting at this one
    // Per-lane byte offsets of the transposing reads inside a stage, for this wavefront's first k-block (a k-block is
    // 16 pair rows) and the first of a lane's two pair rows; the second pair row (4 rows on: same swizzle key) and the
    // k-block go into the instruction's offset field, so a step costs one address add per fragment tile.
    uint32_t a_off[C::TM], b_off[C::TN];
    {
        const int prow = g * 8 + (s16 >> 2);
        static_assert(C::key_a(0) == C::key_a(4) && C::key_b(1) == C::key_b(5), "pair rows 4 apart share a swizzle key");
#pragma unroll
        for (int i = 0; i < C::TM; ++i) {
            const int byte = (wave_m * C::WM + i * 32 + mb * 16 + (s16 & 3) * 4) * 2;
            const int c = byte >> 4, w = byte & 15;
            a_off[i] = (uint32_t)((kk0 * 16 + prow) * C::ROWB_A + ((c ^ C::key_a(prow)) << 4) + w);
        }
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
            const int byte = (wave_n * C::WN + j * 32 + mb * 16 + (s16 & 3) * 4) * 2;
            const int c = byte >> 4, w = byte & 15;
            b_off[j] = (uint32_t)(C::A_BYTES + (kk0 * 16 + prow) * C::ROWB_B + ((c ^ C::key_b(prow)) << 4) + w);
        }
    }
    const uint32_t ring_addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const unsigned char*)ring;
    constexpr int RK = 2 * (C::TM + C::TN);         // LDS reads per k-block
    Walk m = first;
    unsigned step = 0;
    while (m.live) {
        const unsigned b = m.b, v = m.v, tile = m.tile;
        const int nsteps = (int)((m.k_hi - m.k + P - 1) / P);
        f32x16 acc[C::TM][C::TN];
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
            for (int j = 0; j < C::TN; ++j)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
        // Column sums of grad_out (the bias gradient) ride along with the offset whose pairs hold every output row once:
        // the grad_out fragments are multiplied by a fragment of ones as well, so every column of bacc is the sum.  Only
        // the wavefronts of the first column of wave tiles do it, for the first Ci-tile.
        // (not with 128 x 64 or 64 x 128 wave tiles: the extra accumulators do not fit the register budget; the host then sums apart)
        const bool do_bias = C::TM * C::TN <= 4 && bias_partial != nullptr && (int)v == bias_offset && wave_n == 0 && tile < co_tiles;
        f32x16 bacc[C::TM];
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) bacc[i][e] = 0.f;
        // The steps of an item, in two compiled forms: the one with the extra products for the bias gradient runs for
        // the few items that need it, so the other keeps the register allocation and instruction schedule it had.
        auto run_steps = [&](auto with_bias) {
            for (int s = 0; s < nsteps; ++s) {
                asm volatile("" ::: "memory");
                __builtin_amdgcn_s_barrier();           // the loaders saw this step's rows land
                asm volatile("" ::: "memory");
                const uint32_t cur = ring_addr + (step % S) * (uint32_t)C::STAGE_BYTES;
                ++step;
                // Transposing read: in a 16-lane group, lane s supplies the address of 4 adjacent channels of pair row
                // (s / 4) and receives the 4 pair values of channel (group base + s).  Lanes 0-15 / 16-31 cover fragment
                // rows 0-15 / 16-31, the two wave halves take pair rows [0, 8) / [8, 16) of the k-block.  The reads of
                // k-block kk+1 are in flight while k-block kk is multiplied.
                i16x4 fr[2][RK];
                uint32_t a_at[C::TM], b_at[C::TN];
    #pragma unroll
                for (int i = 0; i < C::TM; ++i) a_at[i] = cur + a_off[i];
    #pragma unroll
                for (int j = 0; j < C::TN; ++j) b_at[j] = cur + b_off[j];
                auto read_block = [&](auto kl_c, i16x4 (&dst)[RK]) {        // (the k-block is a compile-time constant)
                    constexpr int kl = decltype(kl_c)::value;
    #pragma unroll
                    for (int i = 0; i < C::TM; ++i) {
                        dst[i * 2] = lds_read_tr16_at<kl * 16 * C::ROWB_A>(a_at[i]);
                        dst[i * 2 + 1] = lds_read_tr16_at<kl * 16 * C::ROWB_A + 4 * C::ROWB_A>(a_at[i]);
                    }
    #pragma unroll
                    for (int j = 0; j < C::TN; ++j) {
                        dst[(C::TM + j) * 2] = lds_read_tr16_at<kl * 16 * C::ROWB_B>(b_at[j]);
                        dst[(C::TM + j) * 2 + 1] = lds_read_tr16_at<kl * 16 * C::ROWB_B + 4 * C::ROWB_B>(b_at[j]);
                    }
                };
                read_block(std::integral_constant<int, 0>{}, fr[0]);
                static_for<NK>([&](auto kk_c) {
                    constexpr int kk = decltype(kk_c)::value;
                    if constexpr (kk + 1 < NK) {
                        read_block(std::integral_constant<int, kk + 1>{}, fr[(kk + 1) & 1]);
                        lds_wait_but<RK>(fr[kk & 1]);
                    } else {
                        lds_wait_but<0>(fr[kk & 1]);
                    }
    #pragma unroll
                    for (int i = 0; i < C::TM; ++i) {
                        const i16x8 af = __builtin_shufflevector(fr[kk & 1][i * 2], fr[kk & 1][i * 2 + 1], 0, 1, 2, 3, 4, 5, 6, 7);
                        if constexpr (decltype(with_bias)::value) mma16<Tag>(bacc[i], af, ones16<Tag>());
    #pragma unroll
                        for (int j = 0; j < C::TN; ++j) {
                            const i16x8 bf = __builtin_shufflevector(fr[kk & 1][(C::TM + j) * 2], fr[kk & 1][(C::TM + j) * 2 + 1], 0, 1, 2, 3, 4, 5, 6, 7);
                            mma16<Tag>(acc[i][j], af, bf);
                        }
                    }
                });
            }
        };
        if constexpr (C::TM * C::TN <= 4) {
            if (do_bias) run_steps(std::true_type{});
            else run_steps(std::false_type{});
        } else {
            run_steps(std::false_type{});
        }
        // partial[b][v][co][ci], fp32
        const unsigned co_tile = tile % co_tiles, ci_tile = tile / co_tiles;
        const int m0 = (int)co_tile * BM, n0 = (int)ci_tile * BN;
        float* dst = partial + (((size_t)b * C::SLICES + (C::KSPLIT ? mw : 0)) * V + v) * ((size_t)Co * Ci);
        typename Tag::type* out = direct ? direct + (size_t)v * Ci : nullptr;      // single voxel block: no partial products
#pragma unroll
        for (int j = 0; j < C::TN; ++j) {
            const int ci = n0 + wave_n * C::WN + j * 32 + l32;
            if (ci >= Ci) continue;
#pragma unroll
            for (int i = 0; i < C::TM; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    int co = m0 + wave_m * C::WM + i * 32 + (e >> 2) * 8 + g * 4 + (e & 3);
                    if (co < Co) {
                        if (out) out[(size_t)co * V * Ci + ci] = from_float<typename Tag::type>(acc[i][j][e]);
                        else dst[(size_t)co * Ci + ci] = acc[i][j][e];
                    }
                }
        }
        if (do_bias && l32 == 0) {                  // bias_partial[block * SLICES + slice][co]
            float* bdst = bias_partial + ((size_t)b * C::SLICES + (C::KSPLIT ? mw : 0)) * Co;
#pragma unroll
            for (int i = 0; i < C::TM; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int co = m0 + wave_m * C::WM + i * 32 + (e >> 2) * 8 + g * 4 + (e & 3);
                    if (co < Co) bdst[co] = bacc[i][e];
                }
        }
        m.k = m.k_hi;                               // on to the next non-empty item
        m.item = after(m.item);
        seek(m);
    }
}

// grad_weight[co][v][ci] = sum over the voxel blocks that have pairs for offset v.  A workgroup owns kReduceElems
// consecutive elements (ci fastest: one 128-byte piece per block for fp32 partials) and cuts the blocks into
// kReduceSlices contiguous ranges, one per group of threads; a slice adds its blocks in ascending order (eight loads in
// flight) and the slice sums are added in ascending order as well, so the result depends on nb alone, not on which
// kernel wrote the partial products.
constexpr int kReduceElems = 32, kReduceSlices = 32;

template <typename T>
__global__ void __launch_bounds__(kReduceElems * kReduceSlices) wgrad_reduce_kernel(const float* __restrict__ partial,
                                                           const uint32_t* __restrict__ bounds, int V, int Ci, int Co,
                                                           unsigned nb, unsigned per_block, T* __restrict__ gw) {
    // `per_block` partial products per voxel block (consecutive in `partial`); nb counts the partial products
    __shared__ float sums[kReduceSlices][kReduceElems];
    const size_t per = (size_t)Co * Ci;
    const size_t total = per * V;
    const int e = threadIdx.x % kReduceElems, slice = threadIdx.x / kReduceElems;
    const unsigned chunk = (nb + kReduceSlices - 1) / kReduceSlices;
    for (size_t base = (size_t)blockIdx.x * kReduceElems; base < total; base += (size_t)gridDim.x * kReduceElems) {
        const size_t i = base + e;
        float s = 0.f;
        if (i < total) {
            int ci = (int)(i % Ci);
            size_t t = i / Ci;
            int v = (int)(t % V);
            int co = (int)(t / V);
            const uint32_t* bd = bounds + (size_t)v * (nb / per_block + 1);
            const float* src = partial + (size_t)v * per + (size_t)co * Ci + ci;
            const size_t stride = (size_t)V * per;
            unsigned b = slice * chunk;
            const unsigned end = b + chunk < nb ? b + chunk : nb;
            for (; b + 8 <= end; b += 8) {
                float x[8];
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    const unsigned blk = (b + q) / per_block;
                    x[q] = bd[blk] < bd[blk + 1] ? src[(size_t)(b + q) * stride] : 0.f;
                }
#pragma unroll
                for (int q = 0; q < 8; ++q) s += x[q];
            }
            for (; b < end; ++b) {
                const unsigned blk = b / per_block;
                if (bd[blk] < bd[blk + 1]) s += src[(size_t)b * stride];
            }
        }
        sums[slice][e] = s;
        __syncthreads();
        if (slice == 0 && i < total) {
            float r = sums[0][e];
#pragma unroll
            for (int q = 1; q < kReduceSlices; ++q) r += sums[q][e];
            gw[i] = from_float<T>(r);
        }
        __syncthreads();
    }
}

// The same sum with one thread per element: 1 KiB contiguous per workgroup and block.  For weights whose rows are not a
// multiple of 128 channels (wider ones take the row-per-wavefront kernel below) and that are not so small that this
// leaves most CUs idle while every thread walks a long list of blocks.  Which kernel runs depends on the problem's shape
// alone, not on which kernel wrote the partial products.
template <typename T>
__global__ void __launch_bounds__(256) wgrad_reduce_flat_kernel(const float* __restrict__ partial,
                                                                const uint32_t* __restrict__ bounds, int V, int Ci, int Co,
                                                                unsigned nb, unsigned per_block, T* __restrict__ gw) {
    const size_t per = (size_t)Co * Ci;
    const size_t total = per * V;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        int ci = (int)(i % Ci);
        size_t t = i / Ci;
        int v = (int)(t % V);
        int co = (int)(t / V);
        const uint32_t* bd = bounds + (size_t)v * (nb / per_block + 1);
        const float* src = partial + (size_t)v * per + (size_t)co * Ci + ci;
        const size_t stride = (size_t)V * per;
        float s = 0.f;
        unsigned b = 0;
        for (; b + 8 <= nb; b += 8) {     // eight independent loads in flight; the sum order stays b-ascending
            float x[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const unsigned blk = (b + q) / per_block;
                x[q] = bd[blk] < bd[blk + 1] ? src[(size_t)(b + q) * stride] : 0.f;
            }
#pragma unroll
            for (int q = 0; q < 8; ++q) s += x[q];
        }
        for (; b < nb; ++b) {
            const unsigned blk = b / per_block;
            if (bd[blk] < bd[blk + 1]) s += src[(size_t)b * stride];
        }
        gw[i] = from_float<T>(s);
    }
}

// The same sum with one wavefront per (co, v) row of the result: which blocks have a partial product for this v is
// one ballot over the block table (64 blocks per turn), so the loads of the partial products depend on nothing but
// that mask and eight of them (VEC floats per lane each) are in flight per lane.  Needs Ci to be a multiple of VEC.
// Sums in ascending block order like the other two kernels: same result bit for bit.
template <typename T, int VEC>
__global__ void __launch_bounds__(256) wgrad_reduce_rows_kernel(const float* __restrict__ partial,
                                                                const uint32_t* __restrict__ bounds, int V, int Ci, int Co,
                                                                unsigned nb, unsigned per_block, T* __restrict__ gw) {
    using vec_t = float __attribute__((ext_vector_type(VEC)));
    const int lane = threadIdx.x & 63;
    const size_t rows = (size_t)Co * V;
    const size_t per = (size_t)Co * Ci;
    const size_t stride = (size_t)V * per;
    const unsigned blocks = nb / per_block;
    for (size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6); row < rows; row += (size_t)gridDim.x * 4) {
        const int v = (int)(row % V);
        const size_t co = row / V;
        const uint32_t* bd = bounds + (size_t)v * (blocks + 1);
        const float* src_row = partial + (size_t)v * per + co * Ci;
        T* dst_row = gw + row * Ci;
        for (int c0 = lane * VEC; c0 < Ci; c0 += 64 * VEC) {
            vec_t s = 0.f;
            for (unsigned blk0 = 0; blk0 < blocks; blk0 += 64) {
                const unsigned mine = blk0 + lane;
                uint64_t live = __ballot(mine < blocks && bd[mine] < bd[mine + 1]);
                while (live) {
                    // up to eight live blocks at a time, ascending
                    unsigned idx[8];
                    int cnt = 0;
#pragma unroll
                    for (int q = 0; q < 8; ++q) {
                        idx[q] = 0;
                        if (live) {
                            idx[q] = blk0 + (unsigned)__builtin_ctzll(live);
                            live &= live - 1;
                            cnt = q + 1;
                        }
                    }
                    for (unsigned sl = 0; sl < per_block; ++sl) {
                        vec_t x[8];
#pragma unroll
                        for (int q = 0; q < 8; ++q)
                            if (q < cnt) x[q] = *reinterpret_cast<const vec_t*>(src_row + (size_t)(idx[q] * per_block + sl) * stride + c0);
#pragma unroll
                        for (int q = 0; q < 8; ++q)
                            if (q < cnt) s += x[q];
                    }
                }
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) dst_row[c0 + e] = from_float<T>(s[e]);
        }
    }
}

constexpr unsigned kReduceSlicedFrom = 32;      // partial products from which the sliced reduction is considered
constexpr unsigned kReduceFlatGroups = 1024;    // ... when the flat kernel would launch fewer workgroups than this

template <typename T>
int launch_reduce(const float* partial, const uint32_t* bounds, int V, int Ci, int Co, unsigned nb, unsigned per_block, T* gw,
                  hipStream_t s) {
    const size_t total = (size_t)Co * V * Ci;
    const bool few_groups = nb >= kReduceSlicedFrom && cdiv(total, 256) < kReduceFlatGroups;
    if (Ci % 128 == 0 && per_block == 1 && !few_groups) {
        unsigned g = cdiv((size_t)Co * V, 4);
        if (g > 65536u) g = 65536u;
        if (Ci % 256 == 0)
            wgrad_reduce_rows_kernel<T, 4><<<g, 256, 0, s>>>(partial, bounds, V, Ci, Co, nb, per_block, gw);
        else
            wgrad_reduce_rows_kernel<T, 2><<<g, 256, 0, s>>>(partial, bounds, V, Ci, Co, nb, per_block, gw);
        FGX_CHECK_LAUNCH("fgx_conv_wgrad(reduce)");
        return FGX_OK;
    }
    if (few_groups) {
        unsigned g = cdiv(total, kReduceElems);
        if (g > 65536u) g = 65536u;
        wgrad_reduce_kernel<T><<<g, kReduceElems * kReduceSlices, 0, s>>>(partial, bounds, V, Ci, Co, nb, per_block, gw);
    } else {
        unsigned g = cdiv(total, 256);
        if (g > 65536u) g = 65536u;
        wgrad_reduce_flat_kernel<T><<<g, 256, 0, s>>>(partial, bounds, V, Ci, Co, nb, per_block, gw);
    }
    FGX_CHECK_LAUNCH("fgx_conv_wgrad(reduce)");
    return FGX_OK;
}

// grad_bias[co] = sum over the voxel blocks (and slices) of their column sums.  A workgroup owns 32 columns; its 32
// groups of 32 threads each add every 32nd slot (eight independent loads in flight), then the group sums are added in
// group order: a fixed order, the same on every run.  `live` is the block table row of the offset the sums were made
// from: a block without a pair there was skipped by the kernel and its slots hold nothing.
template <typename T>
__global__ void __launch_bounds__(1024) bias_reduce_kernel(const float* __restrict__ bias_partial,
                                                           const uint32_t* __restrict__ live, unsigned slots, unsigned slices,
                                                           int Co, T* __restrict__ out) {
    __shared__ float sums[32][33];
    const int c = threadIdx.x & 31, grp = threadIdx.x >> 5;
    const int co = blockIdx.x * 32 + c;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (co < Co) {
        for (unsigned base = grp; base < slots; base += 256) {
            // eight slots at a time, no serial tail: first which of them were written, then their sums
            bool ok[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const unsigned q = base + 32 * k;
                const unsigned blk = (q < slots ? q : base) / slices;
                ok[k] = q < slots && live[blk] < live[blk + 1];
            }
            float t[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) t[k] = ok[k] ? bias_partial[(size_t)(base + 32 * k) * Co + co] : 0.f;
#pragma unroll
            for (int k = 0; k < 8; ++k) acc[k] += t[k];
        }
    }
    sums[grp][c] = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
    __syncthreads();
    if (grp == 0 && co < Co) {
        float s = 0.f;
#pragma unroll
        for (int k = 0; k < 32; ++k) s += sums[k][c];
        out[co] = from_float<T>(s);
    }
}

// grad_weight[:, v, :] = 0 for the offsets v of `mask`: offsets without a single pair when the kernels write
// grad_weight themselves (they skip empty items)
template <typename T>
__global__ void __launch_bounds__(256) zero_offsets_kernel(T* __restrict__ gw, int Co, int V, int Ci, uint32_t mask) {
    const size_t total = (size_t)Co * V * Ci;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const int v = (int)(i / Ci % V);
        if ((mask >> v) & 1u) gw[i] = from_float<T>(0.f);
    }
}

// With a single voxel block there is one partial product per offset: the kernels round it and write grad_weight
// themselves, and the reduction (and the fp32 scratch traffic) is skipped.  Same bits as the two-kernel path.
template <typename T>
int prepare_direct(const SegTable& tab, int V, int Ci, int Co, T* gw, hipStream_t s) {
    uint32_t empty = 0;
    for (int v = 0; v < V; ++v)
        if (tab.seg[v + 1] == tab.seg[v]) empty |= 1u << v;
    if (empty) {
        unsigned g = cdiv((size_t)Co * V * Ci, 256);
        if (g > 4096u) g = 4096u;
        zero_offsets_kernel<T><<<g, 256, 0, s>>>(gw, Co, V, Ci, empty);
        FGX_CHECK_LAUNCH("fgx_conv_wgrad(zero)");
    }
    return FGX_OK;
}

bool dtype_ok(int dtype) { return dtype == FGX_F16 || dtype == FGX_BF16 || dtype == FGX_F32; }

struct Layout {
    unsigned nb;
    size_t bounds_off, partial_off, bias_off, colsum_off, total;
};

// where the bias gradient goes, and the offset whose pairs hold every output row exactly once (-1: none does)
struct BiasOut {
    void* out = nullptr;
    int offset = -1;
};
constexpr int kMaxSlices = 4;

// `slices`: partial products per (voxel block, offset, tile)
Layout layout(size_t n, int V, int Ci, int Co, int block_rows, int slices) {
    Layout L{};
    L.nb = n ? cdiv(n, (size_t)block_rows) : 0u;
    size_t off = 0;
    L.bounds_off = off;
    off = align_up(off + (size_t)V * (L.nb + 1) * sizeof(uint32_t), 256);
    L.partial_off = off;
    off = align_up(off + (size_t)(L.nb ? L.nb : 1) * slices * V * Co * Ci * sizeof(float), 256);
    L.bias_off = off;           // fp32 column sums of grad_out per voxel block and slice
    off = align_up(off + (size_t)(L.nb ? L.nb : 1) * kMaxSlices * Co * sizeof(float), 256);
    L.colsum_off = off;         // scratch of the stand-alone column sum, for the paths that do not fuse it
    off += fgx_colsum_scratch_bytes((size_t)1 << 40, Co);      // its largest size: the row count it serves is the caller's
    L.total = off;
    return L;
}

template <typename Tag, int BM, int BN, int WAVES_M, int WAVES_N>
int launch_wgrad(const void* gout, const void* feats, const uint32_t* sig_i, const uint32_t* sig_o,
                 const uint32_t* given_bounds, const SegTable& tab,
                 const Layout& L, bool small, int V, int Ci, int Co, int block_rows, void* scratch, void* gw, hipStream_t s) {
    using C = WgradCfg<Tag, BM, BN, WAVES_M, WAVES_N>;
    using T = typename Tag::type;
    // the block table depends on the pair lists and block_rows alone: callers that keep it pass it in
    const uint32_t* bounds = given_bounds ? given_bounds : (const uint32_t*)((char*)scratch + L.bounds_off);
    float* partial = (float*)((char*)scratch + L.partial_off);
    if (L.nb > 0) {
        if (!given_bounds) {
            block_bounds_kernel<<<cdiv((size_t)V * (L.nb + 1), 256), 256, 0, s>>>(sig_o, tab, V, L.nb, (unsigned)block_rows,
                                                                                 (uint32_t*)((char*)scratch + L.bounds_off));
            FGX_CHECK_LAUNCH("fgx_conv_wgrad(bounds)");
        }
        const unsigned co_tiles = cdiv(Co, BM), ci_tiles = cdiv(Ci, BN);
        const size_t grid = (size_t)cdiv((size_t)L.nb * V * co_tiles * ci_tiles, kXcds) * kXcds;
        FGX_CHECK_ARG(grid < 0x7FFFFFFFull, "fgx_conv_wgrad: too many work items (%zu); use larger voxel blocks", grid);
        auto kern = wgrad_kernel<Tag, BM, BN, WAVES_M, WAVES_N>;
        static thread_local bool lds_raised = false;   // one raise of the dynamic LDS limit per thread and instantiation
        if (C::lds_bytes > 64 * 1024 && !lds_raised) {
            FGX_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)C::lds_bytes));
            lds_raised = true;
        }
        const bool direct = L.nb == 1;
        if (direct) {
            int rc = prepare_direct<T>(tab, V, Ci, Co, (T*)gw, s);
            if (rc != FGX_OK) return rc;
        }
        kern<<<(unsigned)grid, C::NT, C::lds_bytes, s>>>(
            (const T*)gout, (const T*)feats, sig_i, sig_o, bounds, V, Ci, Co, L.nb, co_tiles, ci_tiles, small, partial,
            direct ? (T*)gw : nullptr);
        FGX_CHECK_LAUNCH("fgx_conv_wgrad");
        if (direct) return FGX_OK;
    }
    return launch_reduce<T>(partial, bounds, V, Ci, Co, L.nb, 1u, (T*)gw, s);
}

// ------------------------------------------------------------------------------------------------
// Balanced item lists for the streaming kernel.  Its items (voxel block, offset, tile) cost what their pair count says:
// the centre offset pairs every row of a block, a corner offset a fraction, and dealt out in a fixed interleave the
// workgroup with the most pairs sets the launch's time (measured on shells: the mean workgroup has 0.4 to 0.85 of the
// largest one's pairs when there are 1 to 16 items per workgroup).  One workgroup builds the lists, longest processing
// time first on two levels so that tiles of one (block, offset) -- which share the rows they gather through an XCD's
// L2 -- stay on one XCD:
//   1. chunks = up to 32 tiles of one (block, offset), cost = tiles x (pairs + kItemFixedCost); sorted by falling cost;
//   2. each chunk goes to the XCD with the least cost so far (one wavefront, in sorted order);
//   3. per XCD (one wavefront each): the chunks' items go, in the same order, to the workgroup of that XCD with the
//      least cost so far; a workgroup's chain links its items in the order they arrived.
// Items without pairs cost nothing and are linked too, so the chains cover every item whatever the pair lists hold.
// ------------------------------------------------------------------------------------------------
constexpr int kItemListMaxChunks = 2048;        // chunks the builder sorts in LDS (by counting ranks: quadratic)
constexpr unsigned kItemListMaxItems = 4096;    // beyond (16 items per workgroup and more) the fixed interleave is balanced
                                                // to within a few per cent, and the one-workgroup builder takes too long
constexpr size_t kItemListMinRows = 2048, kItemListMaxBlocks = 12, kItemListMaxBlocksTiled = 16;
constexpr unsigned kItemListGreedyChunks = 256; // chunks dealt to the XCDs one by one
constexpr unsigned kItemListMaxGroups = 512;    // 64 workgroups per XCD: one lane each
constexpr uint32_t kItemFixedCost = 1280;       // an item's prologue, epilogue and share of the reduction, in pairs

// minimum over the 64 lanes, in every lane: four shifts inside the rows of 16 lanes, then the rows' last lanes are
// passed on (lanes shifted in from outside a row, and rows a step leaves out, take the identity)
__device__ __forceinline__ uint32_t wave_min_u32(uint32_t v) {
#define FGX_MIN_STEP(ctrl, rows)                                                                               \
    {                                                                                                          \
        const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp((int)0xFFFFFFFF, (int)v, ctrl, rows, 0xF, false); \
        v = o < v ? o : v;                                                                                     \
    }
    FGX_MIN_STEP(0x111, 0xF)    // row_shr:1
    FGX_MIN_STEP(0x112, 0xF)    // row_shr:2
    FGX_MIN_STEP(0x114, 0xF)    // row_shr:4
    FGX_MIN_STEP(0x118, 0xF)    // row_shr:8: lane 15 of every row holds the row's minimum
    FGX_MIN_STEP(0x142, 0xA)    // row_bcast:15 into rows 1 and 3
    FGX_MIN_STEP(0x143, 0xC)    // row_bcast:31 into rows 2 and 3: lane 63 holds the minimum
#undef FGX_MIN_STEP
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// minimum over lanes 0 ... 7, in every lane
__device__ __forceinline__ uint32_t first8_min_u32(uint32_t v) {
#define FGX_MIN_STEP(ctrl)                                                                                    \
    {                                                                                                         \
        const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp((int)0xFFFFFFFF, (int)v, ctrl, 0xF, 0xF, false); \
        v = o < v ? o : v;                                                                                    \
    }
    FGX_MIN_STEP(0x111)         // row_shr:1
    FGX_MIN_STEP(0x112)         // row_shr:2
    FGX_MIN_STEP(0x114)         // row_shr:4: lane 7 holds the minimum of lanes 0 ... 7
#undef FGX_MIN_STEP
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 7);
}

__global__ void __launch_bounds__(1024) wgrad_item_lists_kernel(const uint32_t* __restrict__ bounds, int V, unsigned nb,
                                                                unsigned tiles, unsigned groups, uint32_t* __restrict__ out) {
    __shared__ uint32_t key[kItemListMaxChunks];
    __shared__ uint16_t sorted[kItemListMaxChunks];
    __shared__ uint8_t xcd_of[kItemListMaxChunks];
    const unsigned units = nb * (unsigned)V, per_unit = (tiles + 31) / 32, chunks = units * per_unit;
    const unsigned items = units * tiles, per_xcd = groups / kXcds;
    const int tid = threadIdx.x;
    uint32_t* head = out + kItemListHeader;
    uint32_t* next = head + groups;
    auto unit_cost = [&](unsigned u) -> uint32_t {          // per item of unit u = b * V + v
        const unsigned b = u / (unsigned)V, v = u % (unsigned)V;
        const uint32_t cnt = bounds[v * (nb + 1) + b + 1] - bounds[v * (nb + 1) + b];
        return cnt ? cnt + kItemFixedCost : 0u;
    };
    auto chunk_items = [&](unsigned m) -> unsigned {
        const unsigned j = m % per_unit;
        return tiles - 32 * j < 32 ? tiles - 32 * j : 32;
    };
    if (tid == 0) {
        out[0] = groups;
        out[1] = items;
        out[2] = tiles;
        out[3] = kItemListMagic;
    }
    for (unsigned m = tid; m < chunks; m += 1024) key[m] = unit_cost(m / per_unit) * chunk_items(m);
    __syncthreads();
    for (unsigned m = tid; m < chunks; m += 1024) {         // rank by counting: falling cost, ties by index
        const uint32_t mine = key[m];
        unsigned rank = 0;
        for (unsigned j = 0; j < chunks; ++j) {
            const uint32_t other = key[j];
            rank += (other > mine || (other == mine && j < m)) ? 1u : 0u;
        }
        sorted[rank] = (uint16_t)m;
    }
    __syncthreads();
    const int wave = tid >> 6, lane = tid & 63;
    if (wave == 0) {
        // Chunks to XCDs: lane x < 8 keeps XCD x's cost so far (in units of 32 pairs).  The first kItemListGreedyChunks
        // chunks -- the large ones -- go one by one to the least loaded XCD; the tail goes eight at a time, the largest
        // of a round to the least loaded XCD.
        const bool bin = lane < kXcds;
        uint32_t load = 0;
        const unsigned greedy = chunks < kItemListGreedyChunks ? chunks : kItemListGreedyChunks;
        for (unsigned r0 = 0; r0 < greedy; r0 += 64) {
            const unsigned r = r0 + lane;
            const unsigned m = r < greedy ? sorted[r] : 0u;
            const uint32_t cost = r < greedy ? key[m] >> 5 : 0u;
            const unsigned count = greedy - r0 < 64 ? greedy - r0 : 64;
            int mine = 0;
            for (unsigned j = 0; j < count; ++j) {
                const uint32_t c = (uint32_t)__builtin_amdgcn_readlane((int)cost, (int)j);
                const int best = (int)(first8_min_u32((load << 6) | (uint32_t)lane) & 63u);
                if (lane == best) load += c;
                if ((unsigned)lane == j) mine = best;
            }
            if (r < greedy) xcd_of[m] = (uint8_t)mine;
        }
        for (unsigned r0 = greedy; r0 < chunks; r0 += kXcds) {
            unsigned rank = 0;
#pragma unroll
            for (int o = 0; o < kXcds; ++o) {
                const uint32_t other = (uint32_t)__builtin_amdgcn_readlane((int)load, o);
                rank += (other < load || (other == load && o < lane)) ? 1u : 0u;
            }
            if (bin && r0 + rank < chunks) {
                const unsigned m = sorted[r0 + rank];
                xcd_of[m] = (uint8_t)lane;
                load += key[m] >> 5;
            }
        }
    }
    __syncthreads();
    if (wave >= kXcds) return;
    // Wavefront x deals the items of XCD x's chunks, in the same order, each to the least loaded workgroup of the XCD;
    // lane l < per_xcd is workgroup l * kXcds + x (blockIdx % kXcds is the XCD a workgroup lands on).  A workgroup's
    // chain links its items in the order they arrived.
    const bool bin = (unsigned)lane < per_xcd;
    uint32_t load = 0;
    uint32_t tail = kItemListEnd;
    bool any = false;
    for (unsigned r0 = 0; r0 < chunks; r0 += 64) {
        const unsigned r = r0 + lane;
        const unsigned m_l = r < chunks ? sorted[r] : 0u;
        const bool here = r < chunks && xcd_of[m_l] == wave;
        const uint32_t key_l = key[m_l];
        uint64_t todo = __ballot(here);
        while (todo) {
            const int j = __builtin_ctzll(todo);
            todo &= todo - 1;
            const unsigned m = (unsigned)__builtin_amdgcn_readlane((int)m_l, j);
            const unsigned u = m / per_unit, k = chunk_items(m);
            const uint32_t per = (uint32_t)__builtin_amdgcn_readlane((int)key_l, j) / k;
            const unsigned first_item = u * tiles + 32 * (m % per_unit);
            auto take = [&](uint32_t it) {
                if (any) next[tail] = it;
                else head[(unsigned)lane * kXcds + wave] = it;
                any = true;
                tail = it;
                load += per;
            };
            if (k < 8) {
                for (unsigned i = 0; i < k; ++i) {
                    const int best = (int)(wave_min_u32(bin ? (load << 6) | (uint32_t)lane : 0xFFFFFFFFu) & 63u);
                    if (lane == best) take(first_item + i);
                }
            } else {
                // many items of one cost: the least loaded workgroups take one each (what dealing them one by one does
                // unless a single item is smaller than the gaps between the loads), per_xcd at a time
                for (unsigned done = 0; done < k;) {
                    const unsigned now = k - done < per_xcd ? k - done : per_xcd;
                    unsigned rank = 0;
                    for (unsigned o = 0; o < per_xcd; ++o) {
                        const uint32_t other = (uint32_t)__builtin_amdgcn_readlane((int)load, (int)o);
                        rank += (other < load || (other == load && o < (unsigned)lane)) ? 1u : 0u;
                    }
                    if (bin && rank < now) take(first_item + done + rank);
                    done += now;
                }
            }
        }
    }
    if (bin) {
        if (any) next[tail] = kItemListEnd;
        else head[(unsigned)lane * kXcds + wave] = kItemListEnd;
    }
}

// workgroups of a streaming launch on the current device
int stream_groups(unsigned* out) {
    int dev = 0, cus = 0;
    FGX_CHECK_HIP(hipGetDevice(&dev));
    FGX_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    unsigned groups = (unsigned)(cus > 0 ? cus : 256);
    groups = groups / kXcds * kXcds;                      // whole rounds over the XCDs
    if (groups < (unsigned)kXcds) groups = kXcds;
    *out = groups;
    return FGX_OK;
}

// 0 where the lists do not apply (too many items for them to matter, or for the builder)
size_t item_lists_words(size_t n, int V, int Ci, int Co, int tile_rows, int tile_cols, int block_rows, unsigned groups,
                        unsigned* tiles_out, unsigned* nb_out) {
    const size_t nb = cdiv(n, (size_t)block_rows);
    const size_t tiles = (size_t)cdiv(Co, tile_rows) * cdiv(Ci, tile_cols);
    const size_t items = nb * V * tiles, chunks = nb * V * cdiv(tiles, (size_t)32);
    if (tiles_out) *tiles_out = (unsigned)tiles;
    if (nb_out) *nb_out = (unsigned)nb;
    if (items == 0 || items > kItemListMaxItems || chunks > (size_t)kItemListMaxChunks || groups > kItemListMaxGroups) return 0;
    // a launch over fewer voxels is over before the lists have paid for their making
    if (n < kItemListMinRows) return 0;
    // The lists deal by cost alone and scatter the offsets of a voxel block over the XCDs; the fixed order keeps them on
    // one XCD at one time, where they share the block's rows in L2.  With many blocks the fixed order is balanced well
    // enough and the sharing counts for more (252 392 voxels, 32 channels, 16 blocks: 0.061 ms fixed, 0.070 with lists;
    // 1 026 536 voxels, 63 blocks: 0.163 against 0.327; 256 channels, 16 blocks: 0.559 against 0.512).
    // (up to 12 blocks of single-tile items, 16 of several tiles, which share more per block and XCD)
    if (nb > (tiles >= 2 ? kItemListMaxBlocksTiled : kItemListMaxBlocks)) return 0;
    // a workgroup's load is compared as a 26-bit number: the mean load plus the largest item, with a factor of two to spare
    if (((double)items / groups + 1.0) * ((double)block_rows + kItemFixedCost) * 2.0 >= 67108864.0) return 0;
    return (size_t)kItemListHeader + groups + items;
}

template <typename Tag, int BM, int BN>
int launch_wgrad_stream(const void* gout, const void* feats, const uint32_t* sig_i, const uint32_t* sig_o,
                        const uint32_t* given_bounds, const SegTable& tab, const Layout& L, size_t n, size_t n_in, int V, int Ci, int Co, int block_rows,
                        void* scratch, void* gw, BiasOut bias, const uint32_t* lists, hipStream_t s) {
    using C = WStreamCfg<Tag, BM, BN>;
    using T = typename Tag::type;
    // the block table depends on the pair lists and block_rows alone: callers that keep it pass it in
    const uint32_t* bounds = given_bounds ? given_bounds : (const uint32_t*)((char*)scratch + L.bounds_off);
    float* partial = (float*)((char*)scratch + L.partial_off);
    if (L.nb > 0) {
        if (!given_bounds) {
            block_bounds_kernel<<<cdiv((size_t)V * (L.nb + 1), 256), 256, 0, s>>>(sig_o, tab, V, L.nb, (unsigned)block_rows,
                                                                                 (uint32_t*)((char*)scratch + L.bounds_off));
            FGX_CHECK_LAUNCH("fgx_conv_wgrad(bounds)");
        }
        const unsigned co_tiles = cdiv(Co, BM), ci_tiles = cdiv(Ci, BN);
        const size_t items = (size_t)L.nb * V * co_tiles * ci_tiles;
        FGX_CHECK_ARG(items < 0x7FFFFFFFull, "fgx_conv_wgrad: too many work items (%zu); use larger voxel blocks", items);
        unsigned groups = 0;
        int grc = stream_groups(&groups);
        if (grc != FGX_OK) return grc;
        auto kern = wgrad_stream_kernel<Tag, BM, BN>;
        static thread_local bool lds_raised = false;
        if (C::lds_bytes > 64 * 1024 && !lds_raised) {
            FGX_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)C::lds_bytes));
            lds_raised = true;
        }
        const bool direct = L.nb == 1 && C::SLICES == 1;
        if (direct) {
            int rc = prepare_direct<T>(tab, V, Ci, Co, (T*)gw, s);
            if (rc != FGX_OK) return rc;
        }
        float* bias_partial = bias.out ? (float*)((char*)scratch + L.bias_off) : nullptr;
        const unsigned bias_slots = L.nb * C::SLICES;
        kern<<<groups, C::NT, C::lds_bytes, s>>>((const T*)gout, (const T*)feats, sig_i, sig_o, bounds, V, Ci, Co, L.nb, co_tiles,
                                                 ci_tiles, tab.seg[V], (uint32_t)(n * (size_t)Co * sizeof(T)),
                                                 (uint32_t)(n_in * (size_t)Ci * sizeof(T)), partial, direct ? (T*)gw : nullptr,
                                                 bias_partial, bias.offset, lists);
        FGX_CHECK_LAUNCH("fgx_conv_wgrad(stream)");
        if (bias_partial) {
            bias_reduce_kernel<T><<<cdiv((size_t)Co, 32), 1024, 0, s>>>(bias_partial, bounds + (size_t)bias.offset * (L.nb + 1),
                                                                         bias_slots, (unsigned)C::SLICES, Co, (T*)bias.out);
            FGX_CHECK_LAUNCH("fgx_conv_wgrad(bias reduce)");
        }
        if (direct) return FGX_OK;
    }
    return launch_reduce<T>(partial, bounds, V, Ci, Co, L.nb * C::SLICES, (unsigned)C::SLICES, (T*)gw, s);
}

// the streaming kernel: 16-bit types, tiles of 128x128 or 64x64, operands addressable with 32-bit offsets
template <typename Tag>
bool stream_ok(int tile_rows, int tile_cols, size_t n, size_t n_in, int Ci, int Co, uint32_t n_pairs) {
    if (sizeof(typename Tag::type) != 2) return false;
    if (!((tile_rows == 128 && tile_cols == 128) || (tile_rows == 64 && tile_cols == 64) || (tile_rows == 32 && tile_cols == 32) ||
          (tile_rows == 256 && tile_cols == 128) || (tile_rows == 128 && tile_cols == 256)))
        return false;
    // the 32 x 32 tile writes four partial products per voxel block; fgx_wgrad_scratch_bytes leaves room for them only
    // where the table picks that tile (at most 32 channels on a side): anything wider runs the tiled kernel
    if (tile_rows == 32 && (Ci < Co ? Ci : Co) > 32) return false;
    return (double)n * Co * 2 <= (double)kOobOffset && (double)n_in * Ci * 2 <= (double)kOobOffset &&
           (double)n_pairs * 4 + 256 <= (double)kOobOffset;
}

template <typename Tag>
int dispatch_wgrad_stream(int tile_rows, int tile_cols, const void* gout, const void* feats, const uint32_t* sig_i, const uint32_t* sig_o,
                          const uint32_t* given_bounds, const SegTable& tab, const Layout& L, size_t n, size_t n_in, int V, int Ci, int Co, int block_rows,
                          void* scratch, void* gw, BiasOut bias, const uint32_t* lists, hipStream_t s) {
    if constexpr (sizeof(typename Tag::type) == 2) {
        if (tile_cols == 256) return launch_wgrad_stream<Tag, 128, 256>(gout, feats, sig_i, sig_o, given_bounds, tab, L, n, n_in, V, Ci, Co, block_rows, scratch, gw, bias, lists, s);
        if (tile_rows == 256) return launch_wgrad_stream<Tag, 256, 128>(gout, feats, sig_i, sig_o, given_bounds, tab, L, n, n_in, V, Ci, Co, block_rows, scratch, gw, bias, lists, s);
        if (tile_rows == 128) return launch_wgrad_stream<Tag, 128, 128>(gout, feats, sig_i, sig_o, given_bounds, tab, L, n, n_in, V, Ci, Co, block_rows, scratch, gw, bias, lists, s);
        if (tile_rows == 64) return launch_wgrad_stream<Tag, 64, 64>(gout, feats, sig_i, sig_o, given_bounds, tab, L, n, n_in, V, Ci, Co, block_rows, scratch, gw, bias, lists, s);
        return launch_wgrad_stream<Tag, 32, 32>(gout, feats, sig_i, sig_o, given_bounds, tab, L, n, n_in, V, Ci, Co, block_rows, scratch, gw, bias, lists, s);
    } else {
        set_error("fgx_conv_wgrad: the streaming kernel handles 16-bit types only");
        return FGX_ERR_UNSUPPORTED;
    }
}

template <typename Tag>
int dispatch_wgrad(int tile_rows, int tile_cols, const void* gout, const void* feats, const uint32_t* sig_i,
                   const uint32_t* sig_o, const uint32_t* given_bounds, const SegTable& tab, const Layout& L, bool small, int V, int Ci, int Co,
                   int block_rows, void* scratch, void* gw, hipStream_t s) {
#define FGX_TILE(BM, BN, WMv, WNv)          \
    if (tile_rows == BM && tile_cols == BN) \
        return launch_wgrad<Tag, BM, BN, WMv, WNv>(gout, feats, sig_i, sig_o, given_bounds, tab, L, small, V, Ci, Co, block_rows, scratch, gw, s);
    FGX_TILE(128, 128, 2, 2)
    FGX_TILE(64, 64, 2, 2)
    FGX_TILE(32, 32, 1, 1)
#undef FGX_TILE
    set_error("fgx_conv_wgrad: no kernel for tile %dx%d", tile_rows, tile_cols);
    return FGX_ERR_UNSUPPORTED;
}

}  // namespace
}  // namespace fgx

using namespace fgx;

extern "C" {

size_t fgx_wgrad_scratch_bytes(size_t n, int V, int Ci, int Co, int block_rows) {
    if (V < 1 || V > kMaxV || Ci <= 0 || Co <= 0 || block_rows <= 0) return 0;
    // room for the four partial products per block of the pair-splitting 32 x 32 streaming tile wherever it could run
    return layout(n, V, Ci, Co, block_rows, (Ci < Co ? Ci : Co) <= 32 ? 4 : 1).total;
}

size_t fgx_wgrad_block_bounds_count(size_t n, int V, int block_rows) {
    if (V < 1 || V > kMaxV || block_rows <= 0) return 0;
    return (size_t)V * ((size_t)cdiv(n, (size_t)block_rows) + 1);
}

int fgx_wgrad_block_bounds(const uint32_t* sig_o, const uint32_t* seg_host, size_t n, int V, int block_rows,
                           uint32_t* block_bounds, fgx_stream_t stream) {
    FGX_CHECK_ARG(V >= 1 && V <= kMaxV, "fgx_wgrad_block_bounds: bad kernel volume %d", V);
    FGX_CHECK_ARG(block_rows >= 1, "fgx_wgrad_block_bounds: block_rows must be positive, got %d", block_rows);
    FGX_CHECK_ARG(seg_host && block_bounds, "fgx_wgrad_block_bounds: null buffer");
    FGX_CHECK_ARG(n < 0xFFFFFFFFull, "fgx_wgrad_block_bounds: too many rows");
    SegTable tab;
    for (int v = 0; v <= V; ++v) {
        FGX_CHECK_ARG(v == 0 || seg_host[v] >= seg_host[v - 1], "fgx_wgrad_block_bounds: segment table is not monotone");
        tab.seg[v] = seg_host[v];
    }
    for (int v = V + 1; v <= kMaxV; ++v) tab.seg[v] = seg_host[V];
    FGX_CHECK_ARG(seg_host[V] == seg_host[0] || sig_o != nullptr, "fgx_wgrad_block_bounds: null pair list");
    const unsigned nb = cdiv(n, (size_t)block_rows);
    block_bounds_kernel<<<cdiv((size_t)V * (nb + 1), 256), 256, 0, (hipStream_t)stream>>>(sig_o, tab, V, nb, (unsigned)block_rows,
                                                                                         block_bounds);
    FGX_CHECK_LAUNCH("fgx_wgrad_block_bounds");
    return FGX_OK;
}

size_t fgx_wgrad_item_lists_count(size_t n, int V, int Ci, int Co, int tile_rows, int tile_cols, int block_rows) {
    if (V < 1 || V > kMaxV || Ci <= 0 || Co <= 0 || tile_rows <= 0 || tile_cols <= 0 || block_rows <= 0) return 0;
    unsigned groups = 0;
    if (stream_groups(&groups) != FGX_OK) return 0;
    return item_lists_words(n, V, Ci, Co, tile_rows, tile_cols, block_rows, groups, nullptr, nullptr);
}

int fgx_wgrad_item_lists(const uint32_t* block_bounds, size_t n, int V, int Ci, int Co, int tile_rows, int tile_cols,
                         int block_rows, uint32_t* item_lists, fgx_stream_t stream) {
    FGX_CHECK_ARG(V >= 1 && V <= kMaxV && Ci > 0 && Co > 0, "fgx_wgrad_item_lists: bad shape Ci=%d Co=%d V=%d", Ci, Co, V);
    FGX_CHECK_ARG(tile_rows > 0 && tile_cols > 0 && block_rows > 0, "fgx_wgrad_item_lists: bad tile %d x %d or block_rows %d", tile_rows,
                  tile_cols, block_rows);
    FGX_CHECK_ARG(block_bounds && item_lists, "fgx_wgrad_item_lists: null buffer");
    unsigned groups = 0, tiles = 0, nb = 0;
    int rc = stream_groups(&groups);
    if (rc != FGX_OK) return rc;
    const size_t words = item_lists_words(n, V, Ci, Co, tile_rows, tile_cols, block_rows, groups, &tiles, &nb);
    FGX_CHECK_ARG(words > 0, "fgx_wgrad_item_lists: no lists for this shape (fgx_wgrad_item_lists_count says 0)");
    wgrad_item_lists_kernel<<<1, 1024, 0, (hipStream_t)stream>>>(block_bounds, V, nb, tiles, groups, item_lists);
    FGX_CHECK_LAUNCH("fgx_wgrad_item_lists");
    return FGX_OK;
}

int fgx_conv_wgrad(int dtype, const void* grad_out, const void* feats, const uint32_t* sig_i, const uint32_t* sig_o,
                   const uint32_t* seg_host, const uint32_t* block_bounds, size_t n, size_t n_in, int Ci, int Co, int V,
                   int tile_rows, int tile_cols, int block_rows, int streaming, void* scratch, void* grad_weight,
                   void* grad_bias, int bias_offset, fgx_stream_t stream) {
    return fgx_conv_wgrad_lists(dtype, grad_out, feats, sig_i, sig_o, seg_host, block_bounds, nullptr, n, n_in, Ci, Co, V, tile_rows,
                                tile_cols, block_rows, streaming, scratch, grad_weight, grad_bias, bias_offset, stream);
}

int fgx_conv_wgrad_lists(int dtype, const void* grad_out, const void* feats, const uint32_t* sig_i, const uint32_t* sig_o,
                         const uint32_t* seg_host, const uint32_t* block_bounds, const uint32_t* item_lists, size_t n, size_t n_in,
                         int Ci, int Co, int V, int tile_rows, int tile_cols, int block_rows, int streaming, void* scratch,
                         void* grad_weight, void* grad_bias, int bias_offset, fgx_stream_t stream) {
    FGX_CHECK_ARG(item_lists == nullptr || block_bounds != nullptr, "fgx_conv_wgrad_lists: item lists go with the block table they were made from");
    FGX_CHECK_ARG(dtype_ok(dtype), "fgx_conv_wgrad: unknown dtype %d", dtype);
    FGX_CHECK_ARG(Ci > 0 && Co > 0 && V >= 1 && V <= kMaxV, "fgx_conv_wgrad: bad shape Ci=%d Co=%d V=%d", Ci, Co, V);
    FGX_CHECK_ARG(block_rows >= 1, "fgx_conv_wgrad: block_rows must be positive, got %d", block_rows);
    FGX_CHECK_ARG(streaming == 0 || streaming == 1,
                  "fgx_conv_wgrad: streaming must be 0 or 1, got %d (a schedule with stream = 2 is for fgx_conv_wgrad_sweep)", streaming);
    FGX_CHECK_ARG(seg_host && scratch && grad_weight, "fgx_conv_wgrad: null buffer");
    FGX_CHECK_ARG(n < 0xFFFFFFFFull && n_in < 0xFFFFFFFFull, "fgx_conv_wgrad: too many rows");
    const int es = dtype == FGX_F32 ? 4 : 2;
    FGX_CHECK_ARG(((size_t)Ci * es) % 16 == 0 && ((size_t)Co * es) % 16 == 0,
                  "fgx_conv_wgrad: rows of %d / %d elements are not multiples of 16 bytes", Ci, Co);
    FGX_CHECK_ARG(((uintptr_t)scratch & 255) == 0, "fgx_conv_wgrad: scratch must be 256-byte aligned");
    SegTable tab;
    for (int v = 0; v <= V; ++v) {
        FGX_CHECK_ARG(v == 0 || seg_host[v] >= seg_host[v - 1], "fgx_conv_wgrad: segment table is not monotone");
        tab.seg[v] = seg_host[v];
    }
    for (int v = V + 1; v <= kMaxV; ++v) tab.seg[v] = seg_host[V];
    const bool any = seg_host[V] > seg_host[0];
    if (any) {
        FGX_CHECK_ARG(grad_out && feats && sig_i && sig_o, "fgx_conv_wgrad: null buffer");
        FGX_CHECK_ARG((((uintptr_t)grad_out | (uintptr_t)feats) & 15) == 0, "fgx_conv_wgrad: grad_out and feats must be 16-byte aligned");
    }
    const bool stream_f16 = streaming && any && dtype == FGX_F16 && stream_ok<F16>(tile_rows, tile_cols, n, n_in, Ci, Co, tab.seg[V]);
    const bool stream_bf16 = streaming && any && dtype == FGX_BF16 && stream_ok<BF16>(tile_rows, tile_cols, n, n_in, Ci, Co, tab.seg[V]);
    Layout L = layout(any ? n : 0, V, Ci, Co, block_rows, (stream_f16 || stream_bf16) && tile_rows == 32 ? 4 : 1);
    // 32-bit byte offsets into grad_out / feats are enough below 4 GiB
    const bool small = (double)n * Co * es < 4294967296.0 && (double)n_in * Ci * es < 4294967296.0;
    hipStream_t s = (hipStream_t)stream;
    // The bias gradient is the column sum of grad_out.  The streaming kernel makes it on the side when one offset's pairs
    // hold every output row exactly once (the caller says which); every other path runs the stand-alone column sum.
    BiasOut bias;
    if (grad_bias != nullptr) {
        const bool fuse = (stream_f16 || stream_bf16) && tile_rows <= 128 && tile_cols <= 128 && bias_offset >= 0 && bias_offset < V &&
                          (size_t)(tab.seg[bias_offset + 1] - tab.seg[bias_offset]) == n;
        if (fuse) {
            bias.out = grad_bias;
            bias.offset = bias_offset;
        } else {
            int rc = fgx_colsum(dtype, grad_out, n, Co, (char*)scratch + L.colsum_off, grad_bias, stream);
            if (rc != FGX_OK) return rc;
        }
    }
    // (outside the streaming kernel's range the tiled kernel runs)
    if (stream_f16)
        return dispatch_wgrad_stream<F16>(tile_rows, tile_cols, grad_out, feats, sig_i, sig_o, block_bounds, tab, L, n, n_in, V, Ci, Co, block_rows, scratch, grad_weight, bias, item_lists, s);
    if (stream_bf16)
        return dispatch_wgrad_stream<BF16>(tile_rows, tile_cols, grad_out, feats, sig_i, sig_o, block_bounds, tab, L, n, n_in, V, Ci, Co, block_rows, scratch, grad_weight, bias, item_lists, s);
    switch (dtype) {
        case FGX_F16: return dispatch_wgrad<F16>(tile_rows, tile_cols, grad_out, feats, sig_i, sig_o, block_bounds, tab, L, small, V, Ci, Co, block_rows, scratch, grad_weight, s);
        case FGX_BF16: return dispatch_wgrad<BF16>(tile_rows, tile_cols, grad_out, feats, sig_i, sig_o, block_bounds, tab, L, small, V, Ci, Co, block_rows, scratch, grad_weight, s);
        default: return dispatch_wgrad<F32>(tile_rows, tile_cols, grad_out, feats, sig_i, sig_o, block_bounds, tab, L, small, V, Ci, Co, block_rows, scratch, grad_weight, s);
    }
}

}  // extern "C"
