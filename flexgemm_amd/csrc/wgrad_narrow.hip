// Weight gradient for narrow layers (16-bit types, up to 32 channels on both sides) with the gathered rows resident in
// LDS: the counterpart of conv_gemm_narrow.hip, on the same plan (narrow_plan.h).
//
//   grad_weight[co][v][ci] = sum over rows r with a neighbor at offset v of grad_out[r][co] * feats[source(r, v)][ci]
//
// The block-major kernel fetches two 64-byte rows per (row, offset) pair: 4.4 GB cross the L2 for the 0.65 GB that
// configuration 4 (2.67 M voxels, 32 channels) holds, at the fabric's read limit.  Here a chunk of 128 rows that are
// consecutive on a Z-order curve brings its own grad_out rows (8 KiB) and its ~220 distinct source rows into LDS once;
// the voxels are the K dimension, and the transposing LDS read (ds_read_b64_tr_b16), which takes an address per lane,
// does the gather: lane s of a 16-lane group names 4 channels of the row that the plan's table gives for (chunk row,
// offset) and receives 4 rows' values of one channel.  A missing neighbor is the row of zeros.
//
// Workgroup: 4 multiplying wavefronts + 4 loading wavefronts, two LDS buffers, one barrier per chunk (as in the forward
// kernel).  Multiplier w owns the offsets 8 w ... 8 w + 7 (their 32 x 32 accumulators stay in registers over all the
// chunks of the workgroup; offsets from V on multiply zeros) and walks the chunk's 128 rows in eight k-steps of 16; the
// grad_out fragment of a k-step is read once for the eight offsets.  At the end every workgroup writes its partial
// products, and a second kernel adds them in workgroup order (fixed order: same bits on every run).
// A plan with an overflowing chunk (more distinct sources than slots) is not for this kernel: the caller looks at the
// plan's header and takes the block-major kernel then.
#include "wgrad_device.h"
#include "narrow_plan.h"

namespace fgx {
namespace {

constexpr int kNwMult = 4, kNwLoad = 4, kNwThreads = 64 * (kNwMult + kNwLoad);
constexpr int kNwTaps = 8;                                                       // offsets per multiplier
constexpr int kNwGoutBytes = kNarrowRows * 64;                                   // the chunk's grad_out rows
constexpr int kNwBufferBytes = kNarrowRowBufPad + kNwGoutBytes + kNarrowTableBytes;
constexpr size_t kNwLdsBytes = 2 * (size_t)kNwBufferBytes;
constexpr int kNwSrcGroups = kNarrowSlots / 16 / kNwLoad;                        // 7 wave-wide row loads per loader
constexpr int kNwOutGroups = kNarrowRows / 16 / kNwLoad;                         // 2
constexpr int kNwIds = kNwSrcGroups + kNwOutGroups;

template <typename Tag>
__global__ void __launch_bounds__(kNwThreads)
narrow_wgrad_kernel(const typename Tag::type* __restrict__ gout, const typename Tag::type* __restrict__ feats,
                    const unsigned char* __restrict__ plan, uint32_t chunks, uint32_t plan_bytes, uint32_t gout_bytes,
                    uint32_t feats_bytes, int V, int Ci, int Co, float* __restrict__ partial) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool loader = wave >= kNwMult;
    const int src_row_bytes = Ci * 2, out_row_bytes = Co * 2;

    // chunks of this workgroup: XCD x owns the x-th eighth, its workgroups interleave
    const unsigned G = gridDim.x;
    const unsigned xcd = blockIdx.x % kXcds, slot_in_xcd = blockIdx.x / kXcds, per_round = G / kXcds;
    const unsigned per_xcd = (chunks + kXcds - 1) / kXcds;
    const unsigned range_lo = xcd * per_xcd, range_hi = (xcd + 1) * per_xcd < chunks ? (xcd + 1) * per_xcd : chunks;
    const unsigned first = range_lo + slot_in_xcd;

    // the slot of zeros of both buffers
    if (tid < 8) {
        const u32x4 zero = {0u, 0u, 0u, 0u};
        *reinterpret_cast<u32x4*>(lds + (size_t)(tid >> 2) * kNwBufferBytes + kNarrowSlots * 64 + (tid & 3) * 16) = zero;
    }

    const rsrc_t feats_rs = make_rsrc(feats, feats_bytes);
    const rsrc_t gout_rs = make_rsrc(gout, gout_bytes);
    const rsrc_t plan_rs = make_rsrc(plan, plan_bytes);

    // ---- loaders: per chunk, wavefront lw loads the source-row groups (j * 4 + lw), the grad_out-row groups likewise,
    // and every fourth KiB of the table; the row numbers of the next chunk but one are fetched while the loads fly ----
    const int lw = loader ? wave - kNwMult : 0;
    uint32_t ids[kNwIds];
    auto fetch_ids = [&](unsigned chunk) {
        const uint32_t base = (uint32_t)kNarrowHeader + chunk * (uint32_t)kNarrowPlanStride + (uint32_t)kNarrowTableBytes;
#pragma unroll
        for (int j = 0; j < kNwSrcGroups; ++j)
            ids[j] = __builtin_amdgcn_raw_buffer_load_b32(plan_rs, base + (uint32_t)((j * kNwLoad + lw) * 16 + (lane >> 2)) * 4u, 0, 0);
#pragma unroll
        for (int j = 0; j < kNwOutGroups; ++j)
            ids[kNwSrcGroups + j] = __builtin_amdgcn_raw_buffer_load_b32(
                plan_rs, base + (uint32_t)kNarrowSlots * 4u + (uint32_t)((j * kNwLoad + lw) * 16 + (lane >> 2)) * 4u, 0, 0);
    };
    auto enqueue = [&](unsigned chunk, int b) {
        unsigned char* buf = lds + (size_t)b * kNwBufferBytes;
#pragma unroll
        for (int j = 0; j < kNwSrcGroups; ++j) {
            const int group = j * kNwLoad + lw;
            const uint32_t s = (uint32_t)(group * 16 + (lane >> 2));
            const uint32_t piece = (uint32_t)(lane & 3) ^ narrow_piece_key(s);
            const bool live = ids[j] != FGX_EMPTY32 && (int)(piece * 16) < src_row_bytes;
            const uint32_t vo = live ? ids[j] * (uint32_t)src_row_bytes + piece * 16u : kNarrowOob;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(feats_rs, FGX_LDS_PTR(buf + group * 1024), 16, vo, 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < kNwOutGroups; ++j) {
            const int group = j * kNwLoad + lw;
            const uint32_t s = (uint32_t)(group * 16 + (lane >> 2));
            const uint32_t piece = (uint32_t)(lane & 3) ^ narrow_piece_key(s);
            const uint32_t id = ids[kNwSrcGroups + j];
            const bool live = id != FGX_EMPTY32 && (int)(piece * 16) < out_row_bytes;
            const uint32_t vo = live ? id * (uint32_t)out_row_bytes + piece * 16u : kNarrowOob;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(gout_rs, FGX_LDS_PTR(buf + kNarrowRowBufPad + group * 1024), 16, vo, 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < kNarrowTableBytes / 1024 / kNwLoad; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                plan_rs, FGX_LDS_PTR(buf + kNarrowRowBufPad + kNwGoutBytes + (j * kNwLoad + lw) * 1024), 16,
                (uint32_t)kNarrowHeader + chunk * (uint32_t)kNarrowPlanStride + (uint32_t)((j * kNwLoad + lw) * 1024 + lane * 16), 0, 0, 0);
    };

    // ---- multipliers ----
    // Transposing read: in a 16-lane group, lane s supplies the address of 4 adjacent channels of row (s / 4) of a run of
    // four rows and receives those four rows' values of channel (group base + s).  Lanes 0-15 / 16-31 cover channels
    // 0-15 / 16-31, the two wave halves take rows [0, 8) / [8, 16) of a k-step, a second read the rows four further on.
    const int mw = loader ? 0 : wave;
    const int s16 = lane & 15, mb = (lane >> 4) & 1, g = lane >> 5;
    const int q = s16 >> 2;                                                      // row of the run of four
    const int chan_byte = mb * 32 + (s16 & 3) * 8;                               // the lane's 4 channels inside a row
    const uint32_t cpiece = (uint32_t)(chan_byte >> 4), cw = (uint32_t)(chan_byte & 15);
    // The two roles run loops of their own (with the same number of barriers): the multipliers' accumulators then take
    // no registers from the loaders and the other way round.
    if (loader) {
        if (first < range_hi) {
            fetch_ids(first);
            enqueue(first, 0);
            if (first + per_round < range_hi) fetch_ids(first + per_round);
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
            int b = 0;
            for (unsigned chunk = first; chunk < range_hi; chunk += per_round, b ^= 1) {
                const unsigned next = chunk + per_round;
                const bool enqueues = next < range_hi, fetches = next + per_round < range_hi;
                if (enqueues) {
                    enqueue(next, b ^ 1);
                    if (fetches) fetch_ids(next + per_round);
                }
                if (fetches) wait_vmcnt<kNwIds>();
                else wait_vmcnt<0>();
                __syncthreads();
            }
        }
        return;
    }
    f32x16 acc[kNwTaps];
#pragma unroll
    for (int t = 0; t < kNwTaps; ++t)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[t][e] = 0.f;
    if (first < range_hi) {
        __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
        int b = 0;
        for (unsigned chunk = first; chunk < range_hi; chunk += per_round, b ^= 1) {
            const unsigned char* buf = lds + (size_t)b * kNwBufferBytes;
            const unsigned char* gbuf = buf + kNarrowRowBufPad;
            const unsigned char* table = gbuf + kNwGoutBytes;
            // grad_out rows sit in the slots of their chunk row numbers: row r = kk * 16 + g * 8 + q (+ 4) has the
            // piece key (g * 2 (+ 1)) & 3, whatever kk
            const uint32_t g_lo = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const unsigned char*)gbuf +
                                  (uint32_t)((g * 8 + q) * 64) + ((cpiece ^ (uint32_t)((g * 2) & 3)) << 4) + cw;
            const uint32_t g_hi = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const unsigned char*)gbuf +
                                  (uint32_t)((g * 8 + q + 4) * 64) + ((cpiece ^ (uint32_t)((g * 2 + 1) & 3)) << 4) + cw;
            const uint32_t row_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const unsigned char*)buf + cw;
#pragma unroll 1
            for (int kk = 0; kk < kNarrowRows / 16; ++kk) {
                // the table entries of this lane's two rows for the wavefront's eight offsets: 16 bytes each
                const int r0 = kk * 16 + g * 8 + q;
                const u32x4 e_lo = *reinterpret_cast<const u32x4*>(table + r0 * (kNarrowTableStride * 2) + mw * 16);
                const u32x4 e_hi = *reinterpret_cast<const u32x4*>(table + (r0 + 4) * (kNarrowTableStride * 2) + mw * 16);
                i16x4 gfr[2], ffr[16];                                       // grad_out (lo, hi); eight offsets (lo, hi)
                gfr[0] = lds_read_tr16_at<0>(g_lo + (uint32_t)(kk * 16 * 64));
                gfr[1] = lds_read_tr16_at<0>(g_hi + (uint32_t)(kk * 16 * 64));
                auto at = [&](const u32x4& e, int t) -> uint32_t {
                    const uint32_t word = e[t >> 1];
                    const uint32_t off = (t & 1) ? word >> 16 : word & 0xFFFFu;
                    return row_base + (off ^ (cpiece << 4));
                };
#pragma unroll
                for (int t = 0; t < 6; ++t) {                                // (at most 15 reads are counted in flight)
                    ffr[t * 2] = lds_read_tr16_at<0>(at(e_lo, t));
                    ffr[t * 2 + 1] = lds_read_tr16_at<0>(at(e_hi, t));
                }
                // every fragment register is tied to the wait: the compiler must not touch one before it
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(gfr[0]), "+v"(gfr[1]));
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(ffr[0]), "+v"(ffr[1]), "+v"(ffr[2]), "+v"(ffr[3]));
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(ffr[4]), "+v"(ffr[5]), "+v"(ffr[6]), "+v"(ffr[7]));
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(ffr[8]), "+v"(ffr[9]), "+v"(ffr[10]), "+v"(ffr[11]));
#pragma unroll
                for (int t = 6; t < 8; ++t) {
                    ffr[t * 2] = lds_read_tr16_at<0>(at(e_lo, t));
                    ffr[t * 2 + 1] = lds_read_tr16_at<0>(at(e_hi, t));
                }
                const i16x8 gf = __builtin_shufflevector(gfr[0], gfr[1], 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int t = 0; t < 6; ++t) {
                    const i16x8 ff = __builtin_shufflevector(ffr[t * 2], ffr[t * 2 + 1], 0, 1, 2, 3, 4, 5, 6, 7);
                    mma16<Tag>(acc[t], gf, ff);
                }
                asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(ffr[12]), "+v"(ffr[13]), "+v"(ffr[14]), "+v"(ffr[15]));
#pragma unroll
                for (int t = 6; t < 8; ++t) {
                    const i16x8 ff = __builtin_shufflevector(ffr[t * 2], ffr[t * 2 + 1], 0, 1, 2, 3, 4, 5, 6, 7);
                    mma16<Tag>(acc[t], gf, ff);
                }
            }
            __builtin_amdgcn_s_waitcnt(0);
            __syncthreads();
        }
    }
    // partial[workgroup][v][co][ci] (32 x 32 per offset): accumulator element e of lane (l32, g) is co = (e >> 2) * 8 +
    // g * 4 + (e & 3), ci = l32
    {
        const int l32 = lane & 31;
#pragma unroll
        for (int t = 0; t < kNwTaps; ++t) {
            const int v = mw * kNwTaps + t;
            if (v < V) {
                float* dst = partial + ((size_t)blockIdx.x * V + v) * 1024;
#pragma unroll
                for (int e = 0; e < 16; ++e) dst[((e >> 2) * 8 + g * 4 + (e & 3)) * 32 + l32] = acc[t][e];
            }
        }
    }
}

// grad_weight[co][v][ci] = sum over the workgroups' partial products.  A workgroup owns 64 consecutive elements of the
// padded (v, co, ci) tiles; four groups of 64 threads each add a quarter of the partial products in ascending order
// (eight loads in flight), and the four sums are added in ascending order: a fixed order, whatever the timing.
template <typename T>
__global__ void __launch_bounds__(256) narrow_wgrad_reduce_kernel(const float* __restrict__ partial, unsigned groups, int V, int Ci,
                                                                  int Co, T* __restrict__ gw) {
    __shared__ float part[4][64];
    const unsigned i = blockIdx.x * 64 + (threadIdx.x & 63);                     // (v, co, ci) of the padded 32 x 32 tiles
    const unsigned quarter = threadIdx.x >> 6, per = (groups + 3) / 4;
    const unsigned lo = quarter * per, hi = lo + per < groups ? lo + per : groups;
    const size_t stride = (size_t)V * 1024;
    float s = 0.f;
    unsigned w = lo;
    for (; w + 8 <= hi; w += 8) {
        float x[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] = partial[(size_t)(w + j) * stride + i];
#pragma unroll
        for (int j = 0; j < 8; ++j) s += x[j];
    }
    for (; w < hi; ++w) s += partial[(size_t)w * stride + i];
    part[quarter][threadIdx.x & 63] = s;
    __syncthreads();
    if (quarter == 0) {
        const float total = ((part[0][threadIdx.x] + part[1][threadIdx.x]) + part[2][threadIdx.x]) + part[3][threadIdx.x];
        const int v = i >> 10, co = (i >> 5) & 31, ci = i & 31;
        if (co < Co && ci < Ci) gw[((size_t)co * V + v) * Ci + ci] = from_float<T>(total);
    }
}

int narrow_wgrad_groups(unsigned* out) {
    int dev = 0, cus = 0;
    FGX_CHECK_HIP(hipGetDevice(&dev));
    FGX_CHECK_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    unsigned groups = (unsigned)(cus > 0 ? cus : 256);
    groups = groups / kXcds * kXcds;
    if (groups < (unsigned)kXcds) groups = kXcds;
    *out = groups;
    return FGX_OK;
}

template <typename Tag>
int launch_narrow_wgrad(const void* gout, const void* feats, const void* plan, size_t n, size_t n_src, int V, int Ci, int Co,
                        void* scratch, void* gw, hipStream_t s) {
    using T = typename Tag::type;
    unsigned groups = 0;
    int rc = narrow_wgrad_groups(&groups);
    if (rc != FGX_OK) return rc;
    const uint32_t chunks = (uint32_t)((n + kNarrowRows - 1) / kNarrowRows);
    auto kern = narrow_wgrad_kernel<Tag>;
    static thread_local bool raised = false;
    if (!raised) {
        FGX_CHECK_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kNwLdsBytes));
        raised = true;
    }
    kern<<<groups, kNwThreads, kNwLdsBytes, s>>>((const T*)gout, (const T*)feats, (const unsigned char*)plan, chunks,
                                                 (uint32_t)(kNarrowHeader + (size_t)chunks * kNarrowPlanStride),
                                                 (uint32_t)(n * (size_t)Co * 2), (uint32_t)(n_src * (size_t)Ci * 2), V, Ci, Co,
                                                 (float*)scratch);
    FGX_CHECK_LAUNCH("fgx_conv_narrow_wgrad");
    narrow_wgrad_reduce_kernel<T><<<(unsigned)V * 16, 256, 0, s>>>((const float*)scratch, groups, V, Ci, Co, (T*)gw);
    FGX_CHECK_LAUNCH("fgx_conv_narrow_wgrad(reduce)");
    return FGX_OK;
}

}  // namespace
}  // namespace fgx

using namespace fgx;

extern "C" {

size_t fgx_narrow_wgrad_scratch_bytes(int V) {
    if (V < 1 || V > kNwMult * kNwTaps) return 0;
    unsigned groups = 0;
    if (narrow_wgrad_groups(&groups) != FGX_OK) return 0;
    return (size_t)groups * V * 1024 * sizeof(float);
}

int fgx_conv_narrow_wgrad(int dtype, const void* grad_out, const void* feats, const void* plan, size_t n, size_t n_src, int Ci,
                          int Co, int V, void* scratch, void* grad_weight, fgx_stream_t stream) {
    FGX_CHECK_ARG(dtype == FGX_F16 || dtype == FGX_BF16, "fgx_conv_narrow_wgrad: 16-bit types only, got dtype %d", dtype);
    FGX_CHECK_ARG(V >= 1 && V <= kNarrowMaxV && V <= kNwMult * kNwTaps, "fgx_conv_narrow_wgrad: bad kernel volume %d", V);
    FGX_CHECK_ARG(Ci >= 8 && Ci <= 32 && Ci % 8 == 0 && Co >= 8 && Co <= 32 && Co % 8 == 0,
                  "fgx_conv_narrow_wgrad: Ci = %d and Co = %d must be 8, 16, 24 or 32", Ci, Co);
    FGX_CHECK_ARG(n > 0 && n < 0xFFFFFFFFull, "fgx_conv_narrow_wgrad: bad row count %zu", n);
    FGX_CHECK_ARG((double)n * Co * 2 < (double)0xFF000000u && (double)n_src * Ci * 2 < (double)0xFF000000u,
                  "fgx_conv_narrow_wgrad: operand too large for 32-bit offsets");
    FGX_CHECK_ARG(grad_out && feats && plan && scratch && grad_weight, "fgx_conv_narrow_wgrad: null buffer");
    FGX_CHECK_ARG((((uintptr_t)grad_out | (uintptr_t)feats | (uintptr_t)plan | (uintptr_t)scratch) & 15) == 0,
                  "fgx_conv_narrow_wgrad: buffers must be 16-byte aligned");
    FGX_CHECK_ARG(kNarrowHeader + ((n + kNarrowRows - 1) / kNarrowRows) * (size_t)kNarrowPlanStride < 0xFF000000ull,
                  "fgx_conv_narrow_wgrad: plan passes the 32-bit offset range");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == FGX_F16) return launch_narrow_wgrad<F16>(grad_out, feats, plan, n, n_src, V, Ci, Co, scratch, grad_weight, s);
    return launch_narrow_wgrad<BF16>(grad_out, feats, plan, n, n_src, V, Ci, Co, scratch, grad_weight, s);
}

}  // extern "C"
