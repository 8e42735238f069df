// Weight gradient of the submanifold sparse conv on gfx950: a pair-list GEMM per kernel offset.
//
//   grad_weight[co, v, ci] = sum over pairs k of offset v of grad_out[sig_o[k], co] * feats[sig_i[k], ci]
//
// The contraction runs over pairs, i.e. over ROWS of both operands, while MFMA fragments want the
// contraction index contiguous inside a lane.  Rows are therefore staged in LDS pair-major exactly as
// they arrive from memory (coalesced 16-byte stores) and the fragments are assembled with 16/32-bit
// LDS reads down a column ("transpose on read").
//
// Work decomposition: every offset's pair segment is cut into chunks of `chunk_pairs` pairs; one
// workgroup computes one (chunk, Co-tile, Ci-tile) partial product in fp32 and writes it to scratch;
// a second kernel adds an offset's chunks in a fixed order (deterministic) and casts to the output type.
// Equal-sized chunks balance the very unequal segment lengths (the centre offset has N pairs).
#include "fgx_common.h"

namespace fgx {
namespace {

using f16x8 = _Float16 __attribute__((ext_vector_type(8)));
using bf16x8 = __bf16 __attribute__((ext_vector_type(8)));
using f32x16 = float __attribute__((ext_vector_type(16)));
using u32x4 = uint32_t __attribute__((ext_vector_type(4)));
using u16x8 = uint16_t __attribute__((ext_vector_type(8)));

struct F16 { using type = _Float16; using bits = uint16_t; };
struct BF16 { using type = __bf16; using bits = uint16_t; };
struct F32 { using type = float; using bits = uint32_t; };

template <typename T> __device__ __forceinline__ T from_float(float x);
template <> __device__ __forceinline__ _Float16 from_float<_Float16>(float x) { return (_Float16)x; }
template <> __device__ __forceinline__ float from_float<float>(float x) { return x; }
template <> __device__ __forceinline__ __bf16 from_float<__bf16>(float x) {
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    uint16_t h;
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) h = (uint16_t)((u >> 16) | 0x0040u);
    else h = (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
    return __builtin_bit_cast(__bf16, h);
}

constexpr int kMaxV = 32;

struct ChunkTable {
    uint32_t seg[kMaxV + 1];          // pair offsets per kernel offset
    uint32_t chunk_begin[kMaxV + 1];  // first chunk id of every offset
};

// Pair-major staging: stage[p][c], p < PAIRS, c < W (tile width in elements), row pitch padded by
// 16 bytes so that the lane groups of a column read hit different banks.
template <typename Tag, int BM, int BN, int WAVES_M, int WAVES_N>
struct WgradCfg {
    using T = typename Tag::type;
    using B = typename Tag::bits;
    static constexpr int ES = (int)sizeof(T);
    static constexpr int NT = 64 * WAVES_M * WAVES_N;
    static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    static constexpr int TM = WM / 32, TN = WN / 32;
    static constexpr int KV = 16 / ES;              // elements per fragment vector (8 or 4)
    static constexpr int PAIRS = 2 * KV * 2;        // pairs per step: 2 MFMA k-steps of 2 lane groups x KV
    static constexpr int PITCH_A = BM * ES + 16, PITCH_B = BN * ES + 16;   // bytes
    static constexpr int A_CHUNKS = PAIRS * BM * ES / 16, B_CHUNKS = PAIRS * BN * ES / 16;
    static constexpr int A_PER = (A_CHUNKS + NT - 1) / NT, B_PER = (B_CHUNKS + NT - 1) / NT;
    static constexpr size_t lds_bytes = (size_t)2 * PAIRS * (PITCH_A + PITCH_B) + 2 * PAIRS * 2 * 4;
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of 32x32");
};

template <typename Tag> struct Frag;
template <> struct Frag<F16> {
    static __device__ __forceinline__ void mma(f32x16& acc, const u16x8& a, const u16x8& b) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
    }
};
template <> struct Frag<BF16> {
    static __device__ __forceinline__ void mma(f32x16& acc, const u16x8& a, const u16x8& b) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
    }
};

template <typename Tag, int BM, int BN, int WAVES_M, int WAVES_N>
__global__ void __launch_bounds__(64 * WAVES_M * WAVES_N)
wgrad_kernel(const typename Tag::type* __restrict__ gout, const typename Tag::type* __restrict__ feats,
             const uint32_t* __restrict__ sig_i, const uint32_t* __restrict__ sig_o, ChunkTable tab, int V, int Ci,
             int Co, int chunk_pairs, unsigned co_tiles, unsigned ci_tiles, float* __restrict__ partial) {
    using C = WgradCfg<Tag, BM, BN, WAVES_M, WAVES_N>;
    using Bits = typename Tag::bits;
    constexpr int NT = C::NT;
    constexpr int ES = C::ES;

    const unsigned chunk = blockIdx.y;
    const unsigned co_tile = blockIdx.x % co_tiles;
    const unsigned ci_tile = blockIdx.x / co_tiles;
    int v = 0;
    while (v + 1 < V && tab.chunk_begin[v + 1] <= chunk) ++v;
    const uint32_t k_lo = tab.seg[v] + (chunk - tab.chunk_begin[v]) * (uint32_t)chunk_pairs;
    const uint32_t seg_hi = tab.seg[v + 1];
    const uint32_t k_hi = k_lo + (uint32_t)chunk_pairs < seg_hi ? k_lo + (uint32_t)chunk_pairs : seg_hi;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    unsigned char* a_lds = lds_raw;                                     // [2][PAIRS][PITCH_A]
    unsigned char* b_lds = a_lds + 2 * C::PAIRS * C::PITCH_A;           // [2][PAIRS][PITCH_B]
    uint32_t* idx_lds = (uint32_t*)(b_lds + 2 * C::PAIRS * C::PITCH_B); // [2][2][PAIRS]: (o, i) rows per buffer

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const int g = lane >> 5, l32 = lane & 31;
    const int m0 = (int)co_tile * BM, n0 = (int)ci_tile * BN;

    f32x16 acc[C::TM][C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; ++i)
#pragma unroll
        for (int j = 0; j < C::TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    u32x4 a_reg[C::A_PER], b_reg[C::B_PER];
    const unsigned char* gout_b = (const unsigned char*)gout;
    const unsigned char* feats_b = (const unsigned char*)feats;
    constexpr int A_ROW_CHUNKS = BM * ES / 16, B_ROW_CHUNKS = BN * ES / 16;

    // 16-byte chunk `c` of a tile row: columns [c*KV, c*KV+KV) of the tile; zero when the pair is past
    // the chunk end or the columns are past the tensor width.
    auto load_step = [&](uint32_t k0) {
#pragma unroll
        for (int i = 0; i < C::A_PER; ++i) {
            int c = tid + i * NT;
            u32x4 val = {0u, 0u, 0u, 0u};
            if (c < C::A_CHUNKS) {
                int p = c / A_ROW_CHUNKS, ch = c % A_ROW_CHUNKS;
                int col = m0 + ch * C::KV;
                if (k0 + p < k_hi && col < Co) val = *(const u32x4*)(gout_b + ((size_t)sig_o[k0 + p] * Co + col) * ES);
            }
            a_reg[i] = val;
        }
#pragma unroll
        for (int i = 0; i < C::B_PER; ++i) {
            int c = tid + i * NT;
            u32x4 val = {0u, 0u, 0u, 0u};
            if (c < C::B_CHUNKS) {
                int p = c / B_ROW_CHUNKS, ch = c % B_ROW_CHUNKS;
                int col = n0 + ch * C::KV;
                if (k0 + p < k_hi && col < Ci) val = *(const u32x4*)(feats_b + ((size_t)sig_i[k0 + p] * Ci + col) * ES);
            }
            b_reg[i] = val;
        }
    };
    auto store_step = [&](int buf) {
        unsigned char* a_dst = a_lds + buf * C::PAIRS * C::PITCH_A;
        unsigned char* b_dst = b_lds + buf * C::PAIRS * C::PITCH_B;
#pragma unroll
        for (int i = 0; i < C::A_PER; ++i) {
            int c = tid + i * NT;
            if (c < C::A_CHUNKS) *(u32x4*)(a_dst + (c / A_ROW_CHUNKS) * C::PITCH_A + (c % A_ROW_CHUNKS) * 16) = a_reg[i];
        }
#pragma unroll
        for (int i = 0; i < C::B_PER; ++i) {
            int c = tid + i * NT;
            if (c < C::B_CHUNKS) *(u32x4*)(b_dst + (c / B_ROW_CHUNKS) * C::PITCH_B + (c % B_ROW_CHUNKS) * 16) = b_reg[i];
        }
    };
    (void)idx_lds;

    if (k_lo < k_hi) {
        load_step(k_lo);
        store_step(0);
    }
    __syncthreads();
    int it = 0;
    for (uint32_t k0 = k_lo; k0 < k_hi; k0 += C::PAIRS, ++it) {
        const int buf = it & 1;
        const bool more = k0 + C::PAIRS < k_hi;
        if (more) load_step(k0 + C::PAIRS);
        const unsigned char* a_cur = a_lds + buf * C::PAIRS * C::PITCH_A;
        const unsigned char* b_cur = b_lds + buf * C::PAIRS * C::PITCH_B;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            // lane group g of k-step kk owns pairs [(kk*2+g)*KV, +KV)
            const int p0 = (kk * 2 + g) * C::KV;
            if constexpr (ES == 2) {
                u16x8 af[C::TM], bf[C::TN];
#pragma unroll
                for (int i = 0; i < C::TM; ++i)
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        af[i][e] = *(const Bits*)(a_cur + (p0 + e) * C::PITCH_A + (wave_m * C::WM + i * 32 + l32) * 2);
#pragma unroll
                for (int j = 0; j < C::TN; ++j)
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        bf[j][e] = *(const Bits*)(b_cur + (p0 + e) * C::PITCH_B + (wave_n * C::WN + j * 32 + l32) * 2);
#pragma unroll
                for (int i = 0; i < C::TM; ++i)
#pragma unroll
                    for (int j = 0; j < C::TN; ++j) Frag<Tag>::mma(acc[i][j], af[i], bf[j]);
            } else {
                float af[C::TM][4], bf[C::TN][4];
#pragma unroll
                for (int i = 0; i < C::TM; ++i)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        af[i][e] = *(const float*)(a_cur + (p0 + e) * C::PITCH_A + (wave_m * C::WM + i * 32 + l32) * 4);
#pragma unroll
                for (int j = 0; j < C::TN; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        bf[j][e] = *(const float*)(b_cur + (p0 + e) * C::PITCH_B + (wave_n * C::WN + j * 32 + l32) * 4);
#pragma unroll
                for (int i = 0; i < C::TM; ++i)
#pragma unroll
                    for (int j = 0; j < C::TN; ++j)
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][e], bf[j][e], acc[i][j], 0, 0, 0);
            }
        }
        if (more) store_step(buf ^ 1);
        __syncthreads();
    }

    // partial[chunk][co][ci], fp32
    float* dst = partial + (size_t)chunk * Co * Ci;
#pragma unroll
    for (int j = 0; j < C::TN; ++j) {
        const int ci = n0 + wave_n * C::WN + j * 32 + l32;
        if (ci >= Ci) continue;
#pragma unroll
        for (int i = 0; i < C::TM; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                int co = m0 + wave_m * C::WM + i * 32 + (e >> 2) * 8 + g * 4 + (e & 3);
                if (co < Co) dst[(size_t)co * Ci + ci] = acc[i][j][e];
            }
    }
}

// grad_weight[co][v][ci] = sum over the chunks of offset v, in chunk order
template <typename T>
__global__ void __launch_bounds__(256) wgrad_reduce_kernel(const float* __restrict__ partial, ChunkTable tab, int V,
                                                           int Ci, int Co, T* __restrict__ gw) {
    const size_t per = (size_t)Co * Ci;
    const size_t total = per * V;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        int ci = (int)(i % Ci);
        size_t t = i / Ci;
        int v = (int)(t % V);
        int co = (int)(t / V);
        float s = 0.f;
        for (uint32_t c = tab.chunk_begin[v]; c < tab.chunk_begin[v + 1]; ++c) s += partial[(size_t)c * per + (size_t)co * Ci + ci];
        gw[i] = from_float<T>(s);
    }
}

bool dtype_ok(int dtype) { return dtype == FGX_F16 || dtype == FGX_BF16 || dtype == FGX_F32; }

int make_table(const uint32_t* seg_host, int V, int chunk_pairs, ChunkTable* tab) {
    uint32_t chunks = 0;
    for (int v = 0; v < V; ++v) {
        if (seg_host[v + 1] < seg_host[v]) return -1;
        tab->seg[v] = seg_host[v];
        tab->chunk_begin[v] = chunks;
        uint32_t len = seg_host[v + 1] - seg_host[v];
        chunks += (len + (uint32_t)chunk_pairs - 1) / (uint32_t)chunk_pairs;
    }
    tab->seg[V] = seg_host[V];
    tab->chunk_begin[V] = chunks;
    for (int v = V + 1; v <= kMaxV; ++v) { tab->seg[v] = seg_host[V]; tab->chunk_begin[v] = chunks; }
    return (int)chunks;
}

template <typename Tag, int BM, int BN, int WAVES_M, int WAVES_N>
int launch_wgrad(const void* gout, const void* feats, const uint32_t* sig_i, const uint32_t* sig_o, const ChunkTable& tab,
                 int chunks, int V, int Ci, int Co, int chunk_pairs, void* scratch, void* gw, hipStream_t s) {
    using C = WgradCfg<Tag, BM, BN, WAVES_M, WAVES_N>;
    using T = typename Tag::type;
    if (chunks > 0) {
        const unsigned co_tiles = cdiv(Co, BM), ci_tiles = cdiv(Ci, BN);
        dim3 grid(co_tiles * ci_tiles, (unsigned)chunks, 1);
        wgrad_kernel<Tag, BM, BN, WAVES_M, WAVES_N><<<grid, C::NT, C::lds_bytes, s>>>(
            (const T*)gout, (const T*)feats, sig_i, sig_o, tab, V, Ci, Co, chunk_pairs, co_tiles, ci_tiles, (float*)scratch);
        FGX_CHECK_LAUNCH("fgx_conv_wgrad");
    }
    size_t total = (size_t)Co * V * Ci;
    unsigned g = cdiv(total, 256);
    if (g > 65536u) g = 65536u;
    wgrad_reduce_kernel<T><<<g, 256, 0, s>>>((const float*)scratch, tab, V, Ci, Co, (T*)gw);
    FGX_CHECK_LAUNCH("fgx_conv_wgrad(reduce)");
    return FGX_OK;
}

template <typename Tag>
int dispatch_wgrad(int tile_rows, int tile_cols, const void* gout, const void* feats, const uint32_t* sig_i,
                   const uint32_t* sig_o, const ChunkTable& tab, int chunks, int V, int Ci, int Co, int chunk_pairs,
                   void* scratch, void* gw, hipStream_t s) {
#define FGX_TILE(BM, BN, WMv, WNv)               \
    if (tile_rows == BM && tile_cols == BN)      \
        return launch_wgrad<Tag, BM, BN, WMv, WNv>(gout, feats, sig_i, sig_o, tab, chunks, V, Ci, Co, chunk_pairs, scratch, gw, s);
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

size_t fgx_wgrad_scratch_bytes(const uint32_t* seg_host, int V, int Ci, int Co, int chunk_pairs) {
    if (!seg_host || V < 1 || V > kMaxV || Ci <= 0 || Co <= 0 || chunk_pairs <= 0) return 0;
    ChunkTable tab;
    int chunks = make_table(seg_host, V, chunk_pairs, &tab);
    if (chunks < 0) return 0;
    return (size_t)(chunks > 0 ? chunks : 1) * (size_t)Co * (size_t)Ci * sizeof(float);
}

int fgx_conv_wgrad(int dtype, const void* grad_out, const void* feats, const uint32_t* sig_i, const uint32_t* sig_o,
                   const uint32_t* seg_host, size_t n, int Ci, int Co, int V, int tile_rows, int tile_cols, int chunk_pairs,
                   void* scratch, void* grad_weight, fgx_stream_t stream) {
    FGX_CHECK_ARG(dtype_ok(dtype), "fgx_conv_wgrad: unknown dtype %d", dtype);
    FGX_CHECK_ARG(Ci > 0 && Co > 0 && V >= 1 && V <= kMaxV, "fgx_conv_wgrad: bad shape Ci=%d Co=%d V=%d", Ci, Co, V);
    FGX_CHECK_ARG(chunk_pairs >= 64 && chunk_pairs % 64 == 0, "fgx_conv_wgrad: chunk_pairs must be a positive multiple of 64, got %d", chunk_pairs);
    FGX_CHECK_ARG(seg_host && scratch && grad_weight, "fgx_conv_wgrad: null buffer");
    const int es = dtype == FGX_F32 ? 4 : 2;
    FGX_CHECK_ARG(((size_t)Ci * es) % 16 == 0 && ((size_t)Co * es) % 16 == 0,
                  "fgx_conv_wgrad: rows of %d / %d elements are not multiples of 16 bytes", Ci, Co);
    ChunkTable tab;
    int chunks = make_table(seg_host, V, chunk_pairs, &tab);
    FGX_CHECK_ARG(chunks >= 0 && chunks <= 65535, "fgx_conv_wgrad: segment table is not monotone or needs more than 65535 chunks");
    if (chunks > 0) {
        FGX_CHECK_ARG(grad_out && feats && sig_i && sig_o, "fgx_conv_wgrad: null buffer");
        FGX_CHECK_ARG((((uintptr_t)grad_out | (uintptr_t)feats) & 15) == 0, "fgx_conv_wgrad: grad_out and feats must be 16-byte aligned");
    }
    (void)n;
    hipStream_t s = (hipStream_t)stream;
    switch (dtype) {
        case FGX_F16: return dispatch_wgrad<F16>(tile_rows, tile_cols, grad_out, feats, sig_i, sig_o, tab, chunks, V, Ci, Co, chunk_pairs, scratch, grad_weight, s);
        case FGX_BF16: return dispatch_wgrad<BF16>(tile_rows, tile_cols, grad_out, feats, sig_i, sig_o, tab, chunks, V, Ci, Co, chunk_pairs, scratch, grad_weight, s);
        default: return dispatch_wgrad<F32>(tile_rows, tile_cols, grad_out, feats, sig_i, sig_o, tab, chunks, V, Ci, Co, chunk_pairs, scratch, grad_weight, s);
    }
}

}  // extern "C"
