// Device-side pieces shared by the gather-GEMM kernels: vector types, the MFMA wrappers, conversions,
// the vector-memory wait, and the LDS chunk swizzle.
#pragma once
#include "fgx_common.h"

namespace fgx {
namespace {

constexpr int kXcds = 8;

using f16x8 = _Float16 __attribute__((ext_vector_type(8)));
using bf16x8 = __bf16 __attribute__((ext_vector_type(8)));
using f32x4 = float __attribute__((ext_vector_type(4)));
using f32x16 = float __attribute__((ext_vector_type(16)));
using u32x4 = uint32_t __attribute__((ext_vector_type(4)));

#define FGX_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define FGX_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding: vmcnt = imm[3:0] | imm[15:14] << 4,
// expcnt = imm[6:4], lgkmcnt = imm[11:8]; all-ones = unconstrained)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

struct F16 { using type = _Float16; };
struct BF16 { using type = __bf16; };
struct F32 { using type = float; };

template <typename Tag> __device__ __forceinline__ void mma(f32x16& acc, const u32x4& a, const u32x4& b);
template <> __device__ __forceinline__ void mma<F16>(f32x16& acc, const u32x4& a, const u32x4& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
}
template <> __device__ __forceinline__ void mma<BF16>(f32x16& acc, const u32x4& a, const u32x4& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
}
template <> __device__ __forceinline__ void mma<F32>(f32x16& acc, const u32x4& a, const u32x4& b) {
    const f32x4 af = __builtin_bit_cast(f32x4, a);
    const f32x4 bf = __builtin_bit_cast(f32x4, b);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af.x, bf.x, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af.y, bf.y, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af.z, bf.z, acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_32x32x2f32(af.w, bf.w, acc, 0, 0, 0);
}

// activation of the GEMM epilogues (FGX_ACT_* of the public header), applied to the fp32 sum before it is rounded
__device__ __forceinline__ float activate(float x, int act) { return act == FGX_ACT_RELU ? fmaxf(x, 0.f) : x; }

// ReLU mask of a 16-byte piece of eight 16-bit outputs: bit t is set when element t is greater than zero (not zero, not
// negative, not NaN) -- as unsigned numbers those are the patterns 1 ... the encoding of +infinity (LIMIT).
template <uint32_t LIMIT>
__device__ __forceinline__ uint32_t positive_bits16(const u32x4& v) {
    uint32_t bits = 0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const uint32_t x = v[w];
        bits |= (uint32_t)(((x & 0xFFFFu) - 1u) < LIMIT) << (2 * w);
        bits |= (uint32_t)(((x >> 16) - 1u) < LIMIT) << (2 * w + 1);
    }
    return bits;
}
template <typename T> struct PositiveLimit { static constexpr uint32_t value = 0u; };        // fp32: no mask
template <> struct PositiveLimit<_Float16> { static constexpr uint32_t value = 0x7C00u; };
template <> struct PositiveLimit<__bf16> { static constexpr uint32_t value = 0x7F80u; };

template <typename T> __device__ __forceinline__ T from_float(float x);
template <> __device__ __forceinline__ _Float16 from_float<_Float16>(float x) { return (_Float16)x; }
template <> __device__ __forceinline__ float from_float<float>(float x) { return x; }
template <> __device__ __forceinline__ __bf16 from_float<__bf16>(float x) {
    // round to nearest even; NaN stays NaN
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    uint16_t h;
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) h = (uint16_t)((u >> 16) | 0x0040u);
    else h = (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
    return __builtin_bit_cast(__bf16, h);
}
template <typename T> __device__ __forceinline__ float to_float(T x) { return (float)x; }
template <> __device__ __forceinline__ float to_float<__bf16>(__bf16 x) {
    return __builtin_bit_cast(float, (uint32_t)__builtin_bit_cast(uint16_t, x) << 16);
}

// Physical position of logical chunk `chunk` of slab row `row` (CH chunks per row).  The gfx950 LDS has 64 banks of
// 4 bytes: a 256-byte bank line holds two 128-byte rows (four 64-byte rows), and a 128-bit read serves 16 lanes --
// 16 consecutive slab rows at one logical chunk -- per pass.  The XOR key below gives the rows that share a half
// (quarter) of the bank line distinct chunk positions within any 16 consecutive rows, so a fragment read takes the
// same 4.9 cycles as a linear one (measured; a key with period 8 in the row, e.g. row & 7, takes 8.2: two rows of
// every pass then meet in one bank group).
template <int CH> __device__ __forceinline__ int swz_key(int row) {
    return CH == 8 ? ((row >> 1) & 7) : ((row >> 2) & 3);
}
template <int CH> __device__ __forceinline__ int swz(int row, int chunk) {
    return row * (CH * 16) + ((chunk ^ swz_key<CH>(row)) << 4);
}

}  // namespace
}  // namespace fgx
