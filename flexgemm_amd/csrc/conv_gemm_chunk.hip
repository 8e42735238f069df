// Chunk-resident masked implicit GEMM (forward and dgrad) for 16-bit types on gfx950.
//
//   out[row, :] = sum over offsets v present for the row of src[map[row, v], :] x panel_v (+ bias)
//
// The streaming kernel of conv_gemm_stream.hip gathers every (row, offset) pair from memory: ~10 source rows per
// output row, which makes it a kernel of the vector-memory address path and of the L2 - fabric boundary.  Here the
// gather happens in LDS.  A *chunk* is 512 output rows that lie next to each other along a space-filling curve;
// all source rows their neighbors name -- the chunk itself plus a thin halo, ~1.35 rows per output row -- are
// loaded once per K-slab, and the operand fragments of the MFMAs are read from there through per-row indices:
//
//  * one persistent workgroup per CU walks its chunks; per chunk it runs K-slabs (32 channels: 64 bytes per row)
//    outermost, offsets inside; a step is one (slab, offset);
//  * the 8 wavefronts each own 64 of the chunk's rows as four bands of 16 and all 128 columns of the column
//    tile: 4 x 8 accumulators of a 16x16x32 MFMA, kept in registers over all steps of the chunk.  A band none of
//    whose rows has the step's offset is skipped by its wavefront alone: the plan sorts a chunk's rows by offset
//    mask, so present offsets cluster in bands (at the res-512 shell 90 % of the band x offset MFMA work is useful);
//  * a step's weight slab (128 columns x 64 bytes) travels memory -> LDS two steps ahead through a ring of three,
//    one 1 KiB piece per wavefront; its index column (the local row of every position's neighbor, 2 bytes each) comes
//    with it; the source rows of the next slab (or of the next chunk's first slab) are enqueued a few pieces per step
//    into the second of two row buffers.  Every load writes LDS directly, so a wavefront's vector-memory counter
//    sees only its own loads in issue order and "everything issued two steps ago has landed" is one s_waitcnt;
//  * one workgroup barrier per step; the output tile leaves through the row buffer that has just been retired.
//
// The plan (chunk_src, chunk_idx, chunk_out, chunk_band, chunk_nsrc) is made by fgx_chunk_plan_*; its layout is
// described in include/flexgemm_hip.h.
#include <type_traits>

#include "gemm_device.h"

namespace fgx {
namespace {

constexpr uint32_t kChunkOob = 0xFF000000u;   // buffer offset no operand reaches: the load returns zeros

using rsrc_t = __amdgpu_buffer_rsrc_t;

__device__ __forceinline__ rsrc_t chunk_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), (short)0, (int)bytes, 0x00020000);
}

// The four MFMAs of one band and one half of the column blocks, together with the test of the band's bit and the
// branch around them, as ONE assembly statement.  Which bands a wavefront multiplies changes from step to step; with
// the branch in C++ the compiler tracks every accumulator through every merge point and ends up copying accumulators
// around at each of them (an MFMA's result may live in other registers than its addend): hundreds of moves and spills
// per step.  A statement that reads and writes its accumulators whether or not it multiplies has no merge points.
// What the compiler no longer sees is that the statement is an MFMA: the hazards it would pad are kept apart by
// distance -- an accumulator is touched by one statement per step, and read or cleared by other instructions only
// behind wait_mfma_results().
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}
// (the host pass must not see device-only assembly: it would silently drop the kernel's launch stub)
#if defined(__HIP_DEVICE_COMPILE__)
#define FGX_DEVICE_ONLY(...) __VA_ARGS__
#else
#define FGX_DEVICE_ONLY(...)
#endif
#define FGX_MMA_BAND(NAME)                                                                                         \
    FGX_DEVICE_ONLY(asm volatile("s_bitcmp0_b32 %9, %10\n\t"                                                       \
                                 "s_cbranch_scc1 .Lfgx_skip%=\n\t"                                                 \
                                 "v_mfma_f32_16x16x32_" NAME " %0, %4, %8, %0\n\t"                                 \
                                 "v_mfma_f32_16x16x32_" NAME " %1, %5, %8, %1\n\t"                                 \
                                 "v_mfma_f32_16x16x32_" NAME " %2, %6, %8, %2\n\t"                                 \
                                 "v_mfma_f32_16x16x32_" NAME " %3, %7, %8, %3\n"                                    \
                                 ".Lfgx_skip%=:"                                                                    \
                                 : "+v"(c0), "+v"(c1), "+v"(c2), "+v"(c3)                                           \
                                 : "v"(w0), "v"(w1), "v"(w2), "v"(w3), "v"(rows), "s"(bits), "n"(BAND)              \
                                 : "scc");)
template <typename Tag, int BAND>
__device__ __forceinline__ void mma_band(f32x4& c0, f32x4& c1, f32x4& c2, f32x4& c3, const u32x4& w0, const u32x4& w1,
                                         const u32x4& w2, const u32x4& w3, const u32x4& rows, uint32_t bits) {
    if constexpr (sizeof(typename Tag::type) == 2 && __is_same(typename Tag::type, _Float16)) {
        FGX_MMA_BAND("f16")
    } else {
        FGX_MMA_BAND("bf16")
    }
}
#undef FGX_MMA_BAND
// more than the 4 passes of the last MFMA issued, before its result is read or overwritten by other instructions
__device__ __forceinline__ void wait_mfma_results() { FGX_DEVICE_ONLY(asm volatile("s_nop 15\n\ts_nop 7" ::: "memory");) }

struct ChunkCfg {
    static constexpr int CS = FGX_CHUNK_ROWS;            // positions (output rows) per chunk
    static constexpr int SMAX = FGX_CHUNK_SRC_MAX;       // local source rows per chunk
    static constexpr int NW = 8;                         // wavefronts
    static constexpr int BPW = 4;                        // bands per wavefront
    static constexpr int BAND = 16;                      // rows per band (one 16x16x32 MFMA tile)
    static constexpr int BN = 128;                       // columns per column tile
    static constexpr int NCB = BN / 16;                  // 16-column blocks
    static constexpr int SLAB = 64;                      // bytes of K per step and row
    static constexpr int NT = 64 * NW;
    static constexpr int A_BYTES = SMAX * SLAB;
    static constexpr int A_PIECES = SMAX / 16;           // wave-wide 1 KiB loads per row buffer
    static constexpr int B_BYTES = BN * SLAB;
    // Who enqueues what.  A wavefront's vector-memory counter retires in issue order, so a slow load holds back the
    // wait for every later one of the same wavefront; the three kinds of load are therefore kept in different
    // wavefronts, each with the lead its latency needs:
    //   wavefronts 0..3  the weight slabs (L2 hits): two 1 KiB pieces each per step, B_AHEAD steps ahead;
    //   wavefronts 4..6  the source rows of the next K-slab (memory): needed only when that slab begins;
    //   wavefront  7     the index columns, I_AHEAD steps ahead, and the row lists.
    static constexpr int NBW = 4, NRW = 3;
    static constexpr int B_AHEAD = 3, B_RING = 4;
    static constexpr int I_AHEAD = 7, I_RING = 8;
    static constexpr int IDX_BYTES = NW * BAND * BPW * 2;
    static constexpr int SRC_IDS_BYTES = ((SMAX * 4 + 1023) / 1024) * 1024;
    static constexpr int OUT_PITCH = BN * 2 + 16;        // staged output row (16-bit elements)
    static constexpr int OFF_A = 0;
    static constexpr int OFF_B = OFF_A + 2 * A_BYTES;
    static constexpr int OFF_IDX = OFF_B + B_RING * B_BYTES;
    static constexpr int OFF_IDS = OFF_IDX + I_RING * IDX_BYTES;
    static constexpr int OFF_OROW = OFF_IDS + SRC_IDS_BYTES;     // output row of every position of the current item
    static constexpr int LDS_BYTES = OFF_OROW + CS * 4;
    static constexpr int FIRST_A_STEP = 6;               // row loads of the next slab start at this step of a slab ...
    static constexpr int LAND_STEPS = 4;                 // ... and the last of them is issued this many steps before its end
    static constexpr int ROWS_PER_STEP = 2;              // row loads per row-loading wavefront and step
    static constexpr int MAX_ROW_LOADS = (A_PIECES + NRW - 1) / NRW;     // per slab and wavefront
    // fewest offsets (steps per slab) the schedule works with
    static constexpr int MIN_V = FIRST_A_STEP + LAND_STEPS + (MAX_ROW_LOADS + ROWS_PER_STEP - 1) / ROWS_PER_STEP;
    static_assert(CS == NW * BPW * BAND, "a chunk is 8 wavefronts x 4 bands x 16 rows");
    static_assert(IDX_BYTES == 1024, "an index column is one wave-wide 16-byte load");
    static_assert(SMAX % 16 == 0 && NW * BAND * OUT_PITCH <= A_BYTES, "output staging must fit a row buffer");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS");
    static_assert(BN / 16 == 2 * NBW, "two weight-slab pieces per loading wavefront");
    static_assert((B_RING & (B_RING - 1)) == 0 && (I_RING & (I_RING - 1)) == 0 && B_AHEAD < B_RING && I_AHEAD < I_RING, "rings");
};

template <int LO, int HI>
__device__ __forceinline__ void chunk_wait_vmcnt(int n) {
    if constexpr (LO == HI) {
        wait_vmcnt<LO>();
    } else {
        constexpr int MID = (LO + HI) / 2;
        if (n <= MID) chunk_wait_vmcnt<LO, MID>(n);
        else chunk_wait_vmcnt<MID + 1, HI>(n);
    }
}

__device__ __forceinline__ void chunk_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

enum { kRoleB = 0, kRoleRows = 1, kRoleIdx = 2 };

template <typename Tag>
__global__ void __launch_bounds__(ChunkCfg::NT)
gather_gemm_chunk_kernel(const typename Tag::type* __restrict__ src, const typename Tag::type* __restrict__ panel,
                         const typename Tag::type* __restrict__ bias, const uint32_t* __restrict__ chunk_src,
                         const int32_t* __restrict__ chunk_nsrc, const uint16_t* __restrict__ chunk_idx,
                         const uint32_t* __restrict__ chunk_out, const uint32_t* __restrict__ chunk_band,
                         unsigned nchunks, unsigned col_tiles, int slabs, int V, int cols, int cols_pad,
                         uint32_t row_bytes, uint32_t src_bytes, uint32_t panel_bytes, int act,
                         typename Tag::type* __restrict__ out) {
    // (the host pass sees an empty body: it silently drops the launch stub of a kernel whose body it cannot digest)
#if defined(__HIP_DEVICE_COMPILE__)
    using C = ChunkCfg;
    using T = typename Tag::type;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int l16 = lane & 15, g4 = lane >> 4;

    // ---- this workgroup's items: (chunk, column tile), column tiles of a chunk adjacent.  Workgroups are dealt
    // round-robin to the 8 XCDs; XCD x is given a contiguous eighth of the item list, so that chunks which share
    // halo rows share an L2. ----
    const unsigned total = nchunks * col_tiles;
    const unsigned G = gridDim.x;
    unsigned it0, it_end, it_stride;
    if (G % kXcds == 0) {
        const unsigned per_xcd = (total + kXcds - 1) / kXcds;
        const unsigned x = blockIdx.x % kXcds;
        it0 = x * per_xcd + blockIdx.x / kXcds;
        it_end = (x + 1) * per_xcd < total ? (x + 1) * per_xcd : total;
        it_stride = G / kXcds;
    } else {
        it0 = blockIdx.x;
        it_end = total;
        it_stride = G;
    }
    if (it0 >= it_end) return;                      // whole workgroup

    const rsrc_t src_rs = chunk_rsrc(src, src_bytes);
    const rsrc_t panel_rs = chunk_rsrc(panel, panel_bytes);
    const rsrc_t idx_rs = chunk_rsrc(chunk_idx, nchunks * (uint32_t)V * C::IDX_BYTES);
    const rsrc_t ids_rs = chunk_rsrc(chunk_src, nchunks * (uint32_t)C::SMAX * 4u);
    const rsrc_t orow_rs = chunk_rsrc(chunk_out, nchunks * (uint32_t)C::CS * 4u);
    const uint32_t* orow_lds = (const uint32_t*)(lds + C::OFF_OROW);
    const uint32_t* ids_lds = (const uint32_t*)(lds + C::OFF_IDS);

    // ---- per-lane constants ----
    // weight-slab pieces 2 * wave and 2 * wave + 1 of a step: lane -> column 16 * piece + lane / 4, 16-byte piece lane % 4
    const int b_col = (wave & (C::NBW - 1)) * 32 + (lane >> 2);
    const uint32_t b_voff = (uint32_t)(b_col * C::SLAB + (((lane & 3) ^ swz_key<4>(b_col)) << 4));
    // fragment of 16-column block cb: column cb * 16 + l16 (the swizzle key repeats every 16 columns), chunk g4
    const int b_frag = l16 * C::SLAB + ((g4 ^ swz_key<4>(l16)) << 4);
    const uint32_t b_vstride = (uint32_t)slabs * (uint32_t)cols_pad * C::SLAB;      // panel bytes between offsets
    const uint32_t b_qstride = (uint32_t)cols_pad * C::SLAB;                        // ... and between K-slabs

    // ---- a fetch stream: the (item, K-slab, offset) some loads are enqueued for, a fixed number of steps ahead ----
    struct Stream {
        unsigned it;
        int q, v;
        bool live;
        uint32_t soff;      // scalar byte offset of the stream's operand at this position
    };
    auto b_offset = [&](unsigned item, int q, int v) __attribute__((always_inline)) -> uint32_t {
        const unsigned ct = item % col_tiles;
        return (uint32_t)v * b_vstride + (uint32_t)q * b_qstride + ct * (uint32_t)(C::BN * C::SLAB);
    };
    auto i_offset = [&](unsigned item, int v) __attribute__((always_inline)) -> uint32_t { return ((item / col_tiles) * (uint32_t)V + (uint32_t)v) * C::IDX_BYTES; };
    auto advance_b = [&](Stream& p) __attribute__((always_inline)) {
        p.soff += b_vstride;
        if (++p.v < V) return;
        p.v = 0;
        if (++p.q == slabs) {
            p.q = 0;
            if (p.it + it_stride < it_end) p.it += it_stride;
            else p.live = false;            // the stream stays on its last item: loads go on, into slots nobody reads
        }
        p.soff = b_offset(p.it, p.q, 0);
    };
    auto advance_i = [&](Stream& p) __attribute__((always_inline)) {
        p.soff += C::IDX_BYTES;
        if (++p.v < V) return;
        p.v = 0;
        if (++p.q == slabs) {
            p.q = 0;
            if (p.it + it_stride < it_end) p.it += it_stride;
            else p.live = false;
        }
        p.soff = i_offset(p.it, 0);
    };
    // ---- loads ----
    auto fetch_b = [&](const Stream& p, int slot) __attribute__((always_inline)) {                  // weight slab (this wavefront's two pieces)
        unsigned char* dst = lds + C::OFF_B + slot * C::B_BYTES + (wave & (C::NBW - 1)) * 2048;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(panel_rs, FGX_LDS_PTR(dst), 16, b_voff, p.soff, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(panel_rs, FGX_LDS_PTR(dst + 1024), 16, b_voff + 1024u, p.soff, 0, 0);
    };
    auto fetch_idx = [&](const Stream& p, int slot) __attribute__((always_inline)) {                // index column
        __builtin_amdgcn_raw_ptr_buffer_load_lds(idx_rs, FGX_LDS_PTR(lds + C::OFF_IDX + slot * C::IDX_BYTES), 16,
                                                 (uint32_t)(lane * 16), p.soff, 0, 0);
    };
    auto fetch_ids = [&](unsigned c) __attribute__((always_inline)) -> int {                        // the list of source rows of chunk c
        const uint32_t soff = __builtin_amdgcn_readfirstlane(c * (uint32_t)(C::SMAX * 4));
#pragma unroll
        for (int piece = 0; piece < C::SRC_IDS_BYTES / 1024; ++piece)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ids_rs, FGX_LDS_PTR(lds + C::OFF_IDS + piece * 1024), 16,
                                                     (uint32_t)(piece * 1024 + lane * 16), soff, 0, 0);
        return C::SRC_IDS_BYTES / 1024;
    };
    auto fetch_orows = [&](unsigned c) __attribute__((always_inline)) -> int {                      // the output rows of chunk c
        const uint32_t soff = __builtin_amdgcn_readfirstlane(c * (uint32_t)(C::CS * 4));
#pragma unroll
        for (int piece = 0; piece < C::CS * 4 / 1024; ++piece)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(orow_rs, FGX_LDS_PTR(lds + C::OFF_OROW + piece * 1024), 16,
                                                     (uint32_t)(piece * 1024 + lane * 16), soff, 0, 0);
        return C::CS * 4 / 1024;
    };
    // piece j (16 local rows) of K-slab q of the chunk whose source list sits in LDS, into row buffer `buf`
    auto fetch_rows = [&](int j, int q, int buf) __attribute__((always_inline)) {
        const int r = j * 16 + (lane >> 2);
        const uint32_t id = ids_lds[r];
        const uint32_t vo = id == FGX_EMPTY32 ? kChunkOob : id * row_bytes + (uint32_t)(((lane & 3) ^ swz_key<4>(r)) << 4);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(src_rs, FGX_LDS_PTR(lds + C::OFF_A + buf * C::A_BYTES + j * 1024), 16, vo,
                                                 (uint32_t)(q * C::SLAB), 0, 0);
    };

    auto fetch_rows_id = [&](uint32_t id, int j, int q, int buf) __attribute__((always_inline)) {
        const int r = j * 16 + (lane >> 2);
        const uint32_t vo = id == FGX_EMPTY32 ? kChunkOob : id * row_bytes + (uint32_t)(((lane & 3) ^ swz_key<4>(r)) << 4);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(src_rs, FGX_LDS_PTR(lds + C::OFF_A + buf * C::A_BYTES + j * 1024), 16, vo,
                                                 (uint32_t)(q * C::SLAB), 0, 0);
    };

    // ---- accumulators: clearing, and the epilogue of one item: accumulators (+ bias) -> row buffer `buf` -> whole
    // 16-byte pieces of output rows ----
    f32x4 acc[C::BPW][C::NCB];
    auto zero_acc = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int b = 0; b < C::BPW; ++b)
#pragma unroll
            for (int cb = 0; cb < C::NCB; ++cb) acc[b][cb] = f32x4{0.f, 0.f, 0.f, 0.f};
    };
    auto epilogue = [&](unsigned item, int buf) __attribute__((always_inline)) {
        const unsigned ct = item % col_tiles;
        const uint32_t my_row = orow_lds[wave * 64 + lane];
        unsigned char* stage = lds + C::OFF_A + buf * C::A_BYTES + wave * (C::BAND * C::OUT_PITCH);
        const int col0 = (int)ct * C::BN;
        static_for<0, C::BPW>([&](auto bi) __attribute__((always_inline)) {
            constexpr int b = decltype(bi)::value;
            // lane holds row l16 of the band, columns cb * 16 + 4 * g4 + {0..3} of every block cb
            static_for<0, C::NCB>([&](auto cbi) __attribute__((always_inline)) {
                constexpr int cb = decltype(cbi)::value;
                const int cc = cb * 16 + g4 * 4;
                f32x4 bv = {0.f, 0.f, 0.f, 0.f};
                if (bias != nullptr && col0 + cc < cols) {       // (columns come in whole groups of 8)
                    const uint64_t raw = *(const uint64_t*)(bias + col0 + cc);
                    T bq[4];
                    __builtin_memcpy(bq, &raw, 8);
                    bv = f32x4{to_float<T>(bq[0]), to_float<T>(bq[1]), to_float<T>(bq[2]), to_float<T>(bq[3])};
                }
                T pk[4];
                pk[0] = from_float<T>(activate(acc[b][cb][0] + bv.x, act));
                pk[1] = from_float<T>(activate(acc[b][cb][1] + bv.y, act));
                pk[2] = from_float<T>(activate(acc[b][cb][2] + bv.z, act));
                pk[3] = from_float<T>(activate(acc[b][cb][3] + bv.w, act));
                *(uint64_t*)(stage + l16 * C::OUT_PITCH + cc * 2) = __builtin_bit_cast(uint64_t, pk);
            });
            // same wavefront wrote and reads: program order inside the wavefront suffices for LDS
#pragma unroll
            for (int pass = 0; pass < 4; ++pass) {
                const int r = pass * 4 + g4;                      // row of the band
                const int piece = l16;                            // 16-byte piece of its 256 bytes
                const uint32_t orow = (uint32_t)__builtin_amdgcn_ds_bpermute((b * 16 + r) * 4, (int)my_row);
                const int col = col0 + piece * 8;
                if (orow == FGX_EMPTY32 || col >= cols) continue;
                const u32x4 val = *(const u32x4*)(stage + r * C::OUT_PITCH + piece * 16);
                __builtin_nontemporal_store(val, (u32x4*)(out + (size_t)orow * cols + col));
            }
        });
    };
    // which of this wavefront's four bands have offset v: 4 bits per offset, 16 offsets per 64-bit word
    struct BandBits {
        uint64_t lo, hi;        // offsets 0 .. 15, 16 .. 31
    };
    auto band_bits = [&](unsigned item) __attribute__((always_inline)) -> BandBits {
        const unsigned c = item / col_tiles;
        uint32_t bm[C::BPW];
#pragma unroll
        for (int b = 0; b < C::BPW; ++b) bm[b] = __builtin_amdgcn_readfirstlane(chunk_band[(size_t)c * (C::NW * C::BPW) + wave * C::BPW + b]);
        BandBits t{0, 0};
#pragma unroll 1
        for (int v = 0; v < 16; ++v) {
            uint64_t lo = 0, hi = 0;
#pragma unroll
            for (int b = 0; b < C::BPW; ++b) {
                lo |= (uint64_t)((bm[b] >> v) & 1u) << b;
                hi |= (uint64_t)((bm[b] >> (v + 16)) & 1u) << b;
            }
            t.lo |= lo << (v * 4);
            t.hi |= hi << (v * 4);
        }
        return t;
    };
    auto bits_at = [&](const BandBits& t, int v) __attribute__((always_inline)) -> uint32_t {
#ifdef FGX_CHUNK_E_DENSE
        return 15u;
#endif
        const uint64_t w = v < 16 ? t.lo : t.hi;
        return (uint32_t)(w >> ((v & 15) * 4)) & 15u;
    };
    // row fragments of a step: lane (l16, g4) reads 16 bytes of the local row its band's row l16 names, logical chunk g4
    auto read_rows = [&](uint32_t bits, int islot, int buf, u32x4 (&af)[C::BPW]) {
        if (bits == 0) return;
        const unsigned char* A = lds + C::OFF_A + buf * C::A_BYTES;
        const uint64_t ids = *(const uint64_t*)(lds + C::OFF_IDX + islot * C::IDX_BYTES + wave * 128 + l16 * 8);
#pragma unroll
        for (int b = 0; b < C::BPW; ++b) {
            if (!((bits >> b) & 1u)) continue;
#ifdef FGX_CHUNK_E_IDS
            const uint32_t id = (uint32_t)(l16 + 1 + 16 * b) + ((uint32_t)(ids >> (16 * b)) & 0x30u);
#else
            const uint32_t id = (uint32_t)(ids >> (16 * b)) & 0xFFFFu;
#endif
#ifdef FGX_CHUNK_E_NOA
            af[b] = u32x4{id, id, id, id};
#else
            af[b] = *(const u32x4*)(A + id * C::SLAB + ((g4 ^ ((id >> 2) & 3u)) << 4));
#endif
        }
    };

    auto read_rows_ids = [&](uint32_t bits, uint64_t ids, int buf, u32x4 (&af)[C::BPW]) __attribute__((always_inline)) {
        const unsigned char* A = lds + C::OFF_A + buf * C::A_BYTES;
#pragma unroll
        for (int b = 0; b < C::BPW; ++b) {
            if (!((bits >> b) & 1u)) continue;
#ifdef FGX_CHUNK_E_IDS
            const uint32_t id = (uint32_t)(l16 + 1 + 16 * b) + ((uint32_t)(ids >> (16 * b)) & 0x30u);
#else
            const uint32_t id = (uint32_t)(ids >> (16 * b)) & 0xFFFFu;
#endif
#ifdef FGX_CHUNK_E_NOA
            af[b] = u32x4{id, id, id, id};
#else
            af[b] = *(const u32x4*)(A + id * C::SLAB + ((g4 ^ ((id >> 2) & 3u)) << 4));
#endif
        }
    };

    // ---- prologue: the first steps' weight slabs and index columns, the first chunk's lists and first K-slab ----
    Stream fb{it0, 0, 0, true, b_offset(it0, 0, 0)};
    Stream fi{it0, 0, 0, true, i_offset(it0, 0)};
    // (stream position p goes to ring slot p % ring size; the step loop enqueues position t + 1 + AHEAD behind the
    // barrier that opens step t + 1, so positions 0 .. AHEAD are enqueued here)
    for (int k = 0; k <= C::I_AHEAD; ++k) {
        if (k <= C::B_AHEAD) {
            if (wave < C::NBW) fetch_b(fb, k);
            if (fb.live) advance_b(fb);
        }
        if (wave == C::NW - 1) fetch_idx(fi, k);
        if (fi.live) advance_i(fi);
    }
    if (wave == C::NW - 1) {
        (void)fetch_ids(it0 / col_tiles);
        (void)fetch_orows(it0 / col_tiles);
    }
    wait_vmcnt<0>();
    __syncthreads();
    {
        const int pieces = (chunk_nsrc[it0 / col_tiles] + 15) >> 4;
        for (int j = wave; j < pieces; j += C::NW) fetch_rows(j, 0, 0);
    }
    wait_vmcnt<0>();
    __syncthreads();

    // ---- the step loop, once per role ----
    // Loads are enqueued at a constant rate per role (a stream that has run out of items keeps re-fetching its last
    // position into slots nobody reads), so "the loads of step s have landed" is s_waitcnt with a fixed count:
    //   weight slabs   two loads per step, three steps ahead: at most the four of the last two steps may be in flight;
    //   index columns  one load per step, seven steps ahead: at most the last five (a sixth would do for the columns; five makes sure of the row lists, which are enqueued in front of their step's index column and read five steps later),
    //   source rows    waited for all at once, at the barrier that opens the next slab.
    // (Loads and stores of one wavefront retire in issue order, so the output stores of an epilogue in between only
    // make these waits longer.)
    // The loop is rotated by half a step: the MFMAs of a step are split by column blocks into two halves, and the
    // barrier that opens step t + 1 sits between the halves of step t.  Right behind the barrier a wavefront reads
    // step t + 1's fragments from LDS -- the first half's weight fragments into the registers the first half of step
    // t has just freed, the row fragments into the second of two register sets -- and the second half's MFMAs of step
    // t cover those reads' latency; the second half's weight fragments follow when those MFMAs have freed theirs.
    // Taken branches are what a step must not be made of (each costs an instruction-buffer refill; forty of them made
    // a step of ~100 instructions last a thousand cycles), so the step body exists in a few compile-time kinds -- the
    // steps of a slab differ in what they enqueue -- and every kind is straight-line code but for the band tests of the
    // MFMA statements and the rare boundary work of a slab's last step:
    //   kAfterFirst  enqueues for the slab's step 1 (index role: an item's output rows)
    //   kPlain       nothing special
    //   kRowIds      (row role) reads the list entries of the first row loads
    //   kRows        (row role) enqueues row loads and reads the next list entries
    //   kLast        the slab's last step: the one after it opens the next slab (or item)
    enum { kAfterFirst, kPlain, kRowIds, kRows, kLast };
    auto run = [&](auto role_c) __attribute__((always_inline)) {
        constexpr int ROLE = decltype(role_c)::value;
        constexpr int H = C::NCB / 2;
        const int rw = wave - C::NBW;                  // number among the row-loading wavefronts
        const uint32_t bfrag_base = (uint32_t)(C::OFF_B + b_frag);
        const uint32_t idx_lane = (uint32_t)(C::OFF_IDX + wave * 128 + l16 * 8);
        unsigned cur = it0;
        BandBits tab = band_bits(cur);
        uint32_t bits = bits_at(tab, 0);
        u32x4 af[C::BPW], bf[C::NCB];
        read_rows(15u, 0, 0, af);
#pragma unroll
        for (int cb = 0; cb < C::NCB; ++cb) bf[cb] = *(const u32x4*)(lds + bfrag_base + cb * 1024);
        uint64_t ids = *(const uint64_t*)(lds + idx_lane + 1 * C::IDX_BYTES);       // index entries of the step after the current one
        int bslot = 0, islot = 0;      // ring slots of the current step
        int abuf = 0;                  // row buffer of the current K-slab
        uint32_t row_ids[C::ROWS_PER_STEP] = {};   // (row role) local-row list entries of the next step's pieces
        // the row buffer that is not in use is filled with the slab after the current one: its chunk, K-slab and pieces
        bool t_live = slabs > 1 || it0 + it_stride < it_end;
        unsigned t_chunk = slabs > 1 ? it0 / col_tiles : (it0 + it_stride) / col_tiles;
        int t_q = slabs > 1 ? 1 : 0;
        int t_pieces = (ROLE == kRoleRows && t_live) ? (chunk_nsrc[t_chunk] + 15) >> 4 : 0;
        while (true) {
            const unsigned c = cur / col_tiles;
            const unsigned nxt = cur + it_stride;
            const bool has_next = nxt < it_end;
            BandBits tab_next{0, 0};
            if (has_next) tab_next = band_bits(nxt);
            const uint32_t first_bits_next = has_next ? bits_at(tab_next, 0) : 0u;
            zero_acc();
            int q = 0, v = 0;

            auto step = [&](auto kind_c) __attribute__((always_inline)) {
                constexpr int KIND = decltype(kind_c)::value;
                // ---- first half of step (q, v) ----
#ifdef FGX_CHUNK_NO_COMPUTE
                bits = 0;
#endif
                const uint32_t sbits = __builtin_amdgcn_readfirstlane(bits);
                // the next step's row fragments first (their index entries were read a step ago, the rows have been in
                // LDS since the slab began): the first half's MFMAs cover the reads, and the reads stay out of the
                // burst behind the barrier.  Only a slab's last step must wait for the barrier: its rows are the next slab's.
                u32x4 af_next[C::BPW];
                if (KIND != kLast) read_rows_ids(15u, ids, abuf, af_next);
                static_for<0, C::BPW>([&](auto bi) __attribute__((always_inline)) {        // transposed tile: weights first
                    constexpr int b = decltype(bi)::value;
                    mma_band<Tag, b>(acc[b][0], acc[b][1], acc[b][2], acc[b][3], bf[0], bf[1], bf[2], bf[3], af[b], sbits);
                });
                // ---- the step after this one: (e_q, e_v) of chunk e_c ----
                const int e_v = KIND == kLast ? 0 : v + 1;
                bool item_done = false;
                unsigned e_c = c;
                int e_q = q;
                uint32_t bits_n;
                int abuf_n = abuf;
                if (KIND == kLast) {
                    item_done = q + 1 == slabs;
                    e_q = item_done ? 0 : q + 1;
                    e_c = item_done && has_next ? nxt / col_tiles : c;
                    bits_n = item_done ? first_bits_next : bits_at(tab, 0);
                    abuf_n = abuf ^ 1;
                    // a slab begins: the row buffer it does not use is filled with the slab after it
                    const bool ls = e_q + 1 >= slabs;                   // ... which is the first of the item after
                    const unsigned after = (item_done ? nxt : cur) + it_stride;
                    t_live = (!item_done || has_next) && (!ls || after < it_end);
                    t_chunk = ls ? after / col_tiles : e_c;
                    t_q = ls ? 0 : e_q + 1;
                } else {
                    bits_n = bits_at(tab, e_v);
                }
                const int islot_n = (islot + 1) & (C::I_RING - 1);
                const int bslot_n = (bslot + 1) & (C::B_RING - 1);
                // ---- its loads have landed; everybody is done with this step's LDS reads ----
                if (ROLE == kRoleB) wait_vmcnt<4>();
                else if (ROLE == kRoleIdx) wait_vmcnt<5>();
                else if (KIND == kLast) wait_vmcnt<0>();
                __builtin_amdgcn_s_waitcnt(0xC07F);      // lgkmcnt(0): this wavefront's own LDS reads are done, too
                chunk_barrier();
                // ---- its fragments: the first-half weights, the index entries of the step after it.  (Read whether or
                // not a band is present: a test and a branch cost more than the read.) ----
                const unsigned char* Bn = lds + bfrag_base + bslot_n * C::B_BYTES;
                if (KIND == kLast) read_rows_ids(15u, ids, abuf_n, af_next);
#pragma unroll
                for (int cb = 0; cb < H; ++cb) bf[cb] = *(const u32x4*)(Bn + cb * 1024);
                ids = *(const uint64_t*)(lds + idx_lane + ((islot_n + 1) & (C::I_RING - 1)) * C::IDX_BYTES);
                // ---- enqueue (what the step after this one enqueues) ----
                if (ROLE == kRoleB) {
#if !defined(FGX_CHUNK_NO_LOADS)
                    fetch_b(fb, (bslot_n + C::B_AHEAD) & (C::B_RING - 1));
#endif
                    if (fb.live) advance_b(fb);
                } else if (ROLE == kRoleIdx) {
#if !defined(FGX_CHUNK_NO_LOADS)
                    // the item's output rows, once the previous item's epilogue has read its own; the next slab's row list
                    if (KIND == kAfterFirst) {
                        if (e_q == 0) (void)fetch_orows(e_c);
                    }
                    if (KIND == kLast) {
                        if (t_live) (void)fetch_ids(t_chunk);
                    }
                    fetch_idx(fi, (islot_n + C::I_AHEAD) & (C::I_RING - 1));
#endif
                    if (fi.live) advance_i(fi);
                } else {
#if !defined(FGX_CHUNK_NO_LOADS)
                    if (KIND == kLast) {
                        if (t_live) t_pieces = (chunk_nsrc[t_chunk] + 15) >> 4;
                    }
                    // the list entries were read a step ago; the next step's are read now
                    if (KIND == kRows) {
#pragma unroll
                        for (int k = 0; k < C::ROWS_PER_STEP; ++k) {
                            const int j = ((e_v - C::FIRST_A_STEP) * C::ROWS_PER_STEP + k) * C::NRW + rw;
                            if (j < t_pieces && t_live) fetch_rows_id(row_ids[k], j, t_q, abuf_n ^ 1);
                        }
                    }
                    if (KIND == kRows || KIND == kRowIds) {
#pragma unroll
                        for (int k = 0; k < C::ROWS_PER_STEP; ++k) {
                            const int j = ((e_v + 1 - C::FIRST_A_STEP) * C::ROWS_PER_STEP + k) * C::NRW + rw;
                            if (j < t_pieces && t_live) row_ids[k] = ids_lds[j * 16 + (lane >> 2)];
                        }
                    }
#endif
                }
                // ---- second half of step (q, v) ----
                static_for<0, C::BPW>([&](auto bi) __attribute__((always_inline)) {
                    constexpr int b = decltype(bi)::value;
                    mma_band<Tag, b>(acc[b][4], acc[b][5], acc[b][6], acc[b][7], bf[4], bf[5], bf[6], bf[7], af[b], sbits);
                });
                // ---- the rest of the next step's fragments ----
#pragma unroll
                for (int cb = H; cb < C::NCB; ++cb) bf[cb] = *(const u32x4*)(Bn + cb * 1024);
                // ---- on ----
#pragma unroll
                for (int b = 0; b < C::BPW; ++b) af[b] = af_next[b];
                bits = bits_n;
                bslot = bslot_n;
                islot = islot_n;
                abuf = abuf_n;
                v = e_v;
                q = KIND == kLast ? q + 1 : q;
            };
            // the steps of a slab by kind (the row role enqueues from FIRST_A_STEP on, and reads list entries one step before)
            constexpr int kRowSteps = (C::MAX_ROW_LOADS + C::ROWS_PER_STEP - 1) / C::ROWS_PER_STEP;
            for (int qq = 0; qq < slabs; ++qq) {
                step(std::integral_constant<int, kAfterFirst>{});                      // v = 0
                if (ROLE == kRoleRows) {
                    while (v < C::FIRST_A_STEP - 2) step(std::integral_constant<int, kPlain>{});
                    step(std::integral_constant<int, kRowIds>{});                      // v = FIRST_A_STEP - 2: e_v + 1 = FIRST_A_STEP
                    for (int k = 0; k < kRowSteps; ++k) step(std::integral_constant<int, kRows>{});
                }
                while (v < V - 1) step(std::integral_constant<int, kPlain>{});
                step(std::integral_constant<int, kLast>{});                            // v = V - 1
            }
            // ---- the item's tile leaves through the row buffer its last K-slab used: nobody reads that buffer behind the
            // barrier that opened the next item's first step, and the row loads that refill it come several steps later ----
            wait_mfma_results();
#ifndef FGX_CHUNK_NO_EPILOGUE
            epilogue(cur, abuf ^ 1);
#endif
            if (!has_next) break;
            cur = nxt;
            tab = tab_next;
        }
        wait_vmcnt<0>();
    };
    if (wave < C::NBW) run(std::integral_constant<int, kRoleB>{});
    else if (wave < C::NBW + C::NRW) run(std::integral_constant<int, kRoleRows>{});
    else run(std::integral_constant<int, kRoleIdx>{});
#endif
}

template <typename Tag>
int launch_chunk(const void* src, const void* panel, const void* bias, const uint32_t* chunk_src, const int32_t* chunk_nsrc,
                 const uint16_t* chunk_idx, const uint32_t* chunk_out, const uint32_t* chunk_band, size_t nchunks,
                 size_t n_src, int K, int cols, int V, int max_groups, int act, void* out, hipStream_t s) {
    using C = ChunkCfg;
    using T = typename Tag::type;
    auto kern = gather_gemm_chunk_kernel<Tag>;
    static thread_local bool raised = false;
    if (!raised) {
        FGX_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, C::LDS_BYTES));
        raised = true;
    }
    if (max_groups <= 0) {
        int dev = 0, cus = 0;
        FGX_CHECK_HIP(hipGetDevice(&dev));
        FGX_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
        max_groups = cus > 0 ? cus : 256;
    }
    const int cols_pad = (int)align_up((size_t)cols, (size_t)C::BN);
    const unsigned col_tiles = (unsigned)(cols_pad / C::BN);
    const size_t total = nchunks * col_tiles;
    const unsigned groups = (unsigned)(total < (size_t)max_groups ? total : (size_t)max_groups);
    const int slabs = K * (int)sizeof(T) / C::SLAB;
    kern<<<groups, C::NT, C::LDS_BYTES, s>>>((const T*)src, (const T*)panel, (const T*)bias, chunk_src, chunk_nsrc, chunk_idx,
                                            chunk_out, chunk_band, (unsigned)nchunks, col_tiles, slabs, V, cols, cols_pad,
                                            (uint32_t)(K * sizeof(T)), (uint32_t)(n_src * (size_t)K * sizeof(T)),
                                            (uint32_t)((size_t)V * slabs * cols_pad * C::SLAB), act, (T*)out);
    FGX_CHECK_LAUNCH("fgx_conv_gather_gemm_chunk");
    return FGX_OK;
}

}  // namespace
}  // namespace fgx

using namespace fgx;

extern "C" int fgx_conv_gather_gemm_chunk_supported(int dtype, size_t n_src, int K, int cols, int V) {
    if (dtype != FGX_F16 && dtype != FGX_BF16) return 0;
    if (K <= 0 || cols <= 0 || (K * 2) % ChunkCfg::SLAB != 0 || cols % 8 != 0) return 0;
    if (V < ChunkCfg::MIN_V || V > 32) return 0;
    if (n_src * (size_t)K * 2 > kChunkOob) return 0;
    const size_t slabs = (size_t)K * 2 / ChunkCfg::SLAB;
    if ((size_t)V * slabs * align_up((size_t)cols, (size_t)ChunkCfg::BN) * ChunkCfg::SLAB > kChunkOob) return 0;
    return 1;
}

extern "C" int fgx_conv_gather_gemm_chunk(int dtype, const void* src, const void* panel, const void* bias,
                                          const uint32_t* chunk_src, const int32_t* chunk_nsrc, const uint16_t* chunk_idx,
                                          const uint32_t* chunk_out, const uint32_t* chunk_band, size_t nchunks,
                                          size_t n_src, int K, int cols, int V, int max_groups, int activation, void* out,
                                          fgx_stream_t stream) {
    FGX_CHECK_ARG(activation == FGX_ACT_NONE || activation == FGX_ACT_RELU, "fgx_conv_gather_gemm_chunk: unknown activation %d", activation);
    FGX_CHECK_ARG(dtype == FGX_F16 || dtype == FGX_BF16, "fgx_conv_gather_gemm_chunk: 16-bit element types only (got dtype %d)", dtype);
    FGX_CHECK_ARG(K > 0 && cols > 0 && V >= 1 && V <= 32, "fgx_conv_gather_gemm_chunk: bad shape K=%d cols=%d V=%d", K, cols, V);
    if (nchunks == 0) return FGX_OK;
    if (!fgx_conv_gather_gemm_chunk_supported(dtype, n_src, K, cols, V)) {
        set_error("fgx_conv_gather_gemm_chunk: shape not covered (rows must be whole 64-byte slabs, columns a multiple of 8, "
                  "%d <= V <= 32, operands below 4 GB): K=%d cols=%d V=%d", ChunkCfg::MIN_V, K, cols, V);
        return FGX_ERR_UNSUPPORTED;
    }
    FGX_CHECK_ARG(src && panel && chunk_src && chunk_nsrc && chunk_idx && chunk_out && chunk_band && out,
                  "fgx_conv_gather_gemm_chunk: null buffer");
    FGX_CHECK_ARG((((uintptr_t)src | (uintptr_t)panel | (uintptr_t)chunk_src | (uintptr_t)chunk_idx | (uintptr_t)out) & 15) == 0,
                  "fgx_conv_gather_gemm_chunk: src, panel, chunk_src, chunk_idx and out must be 16-byte aligned");
    FGX_CHECK_ARG(nchunks * (size_t)V * ChunkCfg::IDX_BYTES <= kChunkOob && nchunks * (size_t)ChunkCfg::SMAX * 4 <= kChunkOob,
                  "fgx_conv_gather_gemm_chunk: plan exceeds the 32-bit offset range");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FGX_F16)
        return launch_chunk<F16>(src, panel, bias, chunk_src, chunk_nsrc, chunk_idx, chunk_out, chunk_band, nchunks, n_src, K, cols, V, max_groups, activation, out, s);
    return launch_chunk<BF16>(src, panel, bias, chunk_src, chunk_nsrc, chunk_idx, chunk_out, chunk_band, nchunks, n_src, K, cols, V, max_groups, activation, out, s);
}
