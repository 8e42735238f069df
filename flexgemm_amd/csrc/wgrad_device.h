// Device-side pieces shared by the weight-gradient kernels (wgrad_gemm.hip, wgrad_sweep.hip): vector types, the
// transposing LDS read with its hand-placed waits, the MFMA wrappers, buffer resources.
#pragma once
#include <type_traits>

#include "fgx_common.h"

namespace fgx {
namespace {

using f16x8 = _Float16 __attribute__((ext_vector_type(8)));
using bf16x8 = __bf16 __attribute__((ext_vector_type(8)));
using f32x16 = float __attribute__((ext_vector_type(16)));
using u32x4 = uint32_t __attribute__((ext_vector_type(4)));
using i16x4 = short __attribute__((ext_vector_type(4)));
using i16x8 = short __attribute__((ext_vector_type(8)));

struct F16 { using type = _Float16; };
struct BF16 { using type = __bf16; };
struct F32 { using type = float; };

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
constexpr int kXcds = 8;
// Balanced item lists of the streaming weight gradient: words [0..3] = {workgroups, items, tiles per (block, offset),
// kItemListMagic}, then head[workgroups], then next[items]; kItemListEnd closes a chain.
constexpr uint32_t kItemListEnd = 0xFFFFFFFFu, kItemListMagic = 0x4C495354u;
constexpr int kItemListHeader = 4;

#define FGX_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define FGX_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

struct SegTable {
    uint32_t seg[kMaxV + 1];   // pair offsets per kernel offset
};

// Transposing LDS read, issued as inline assembly: through the compiler builtin every such read is preceded by a
// conservative s_waitcnt vmcnt(0) (the compiler cannot tell it apart from the LDS areas the in-flight direct-to-LDS
// loads are filling), which would drain the whole ring each step.  The price is that the result must be waited
// for by hand: lds_wait_all() below ties the fragment registers to an s_waitcnt lgkmcnt(0).
__device__ __forceinline__ i16x4 lds_read_tr16(const unsigned char* p) {
    const uint32_t addr = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const unsigned char*)p;
    i16x4 r;
    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(r) : "v"(addr));
    return r;
}
// the same with the address given as an LDS byte address plus a constant that goes into the instruction's offset field
template <int OFFSET>
__device__ __forceinline__ i16x4 lds_read_tr16_at(uint32_t addr) {
    static_assert(OFFSET >= 0 && OFFSET < 65536, "the offset field is 16 bits wide");
    i16x4 r;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFFSET));
    return r;
}
template <int N>
__device__ __forceinline__ void lds_wait_all(i16x4 (&r)[N]) {
    static_assert(N % 4 == 0, "fragments come in groups of four registers pairs");
#pragma unroll
    for (int i = 0; i < N; i += 4)
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[i]), "+v"(r[i + 1]), "+v"(r[i + 2]), "+v"(r[i + 3]));
}

template <typename Tag> __device__ __forceinline__ void mma16(f32x16& acc, const i16x8& a, const i16x8& b);
template <> __device__ __forceinline__ void mma16<F16>(f32x16& acc, const i16x8& a, const i16x8& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
}
template <> __device__ __forceinline__ void mma16<BF16>(f32x16& acc, const i16x8& a, const i16x8& b) {
    acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
}
template <> __device__ __forceinline__ void mma16<F32>(f32x16&, const i16x8&, const i16x8&) {}

// eight ones in the 16-bit type, as a fragment
template <typename Tag> __device__ __forceinline__ i16x8 ones16() {
    constexpr short one = sizeof(typename Tag::type) == 2 && __is_same(typename Tag::type, _Float16) ? (short)0x3C00 : (short)0x3F80;
    return i16x8{one, one, one, one, one, one, one, one};
}

constexpr uint32_t kOobOffset = 0xFF000000u;

using rsrc_t = __amdgpu_buffer_rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void* p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), (short)0, (int)bytes, 0x00020000);
}

// f(integral_constant<int, 0>), ..., f(integral_constant<int, N - 1>): a loop whose counter is a compile-time constant
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<N, I + 1>(f);
    }
}

// wait until the LDS reads before the newest N have returned; the registers are tied to the wait so that the
// compiler cannot move their first use above it
template <int N, int R>
__device__ __forceinline__ void lds_wait_but(i16x4 (&r)[R]) {
    static_assert(N >= 0 && N < 16 && R % 4 == 0, "lgkmcnt is a 4-bit counter");
#if defined(__HIP_DEVICE_COMPILE__)   // (the host pass only needs the kernel's signature; it has no such registers)
#pragma unroll
    for (int i = 0; i < R; i += 4)
        asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(r[i]), "+v"(r[i + 1]), "+v"(r[i + 2]), "+v"(r[i + 3]) : "n"(N));
#endif
}

// bounds[v * (nb + 1) + b] = first pair of offset v whose output row is >= b * block_rows
__global__ void __launch_bounds__(256) block_bounds_kernel(const uint32_t* __restrict__ sig_o, SegTable tab, int V,
                                                           unsigned nb, unsigned block_rows,
                                                           uint32_t* __restrict__ bounds) {
    const unsigned t = blockIdx.x * 256 + threadIdx.x;
    if (t >= (unsigned)V * (nb + 1)) return;
    const unsigned v = t / (nb + 1), b = t % (nb + 1);
    uint32_t lo = tab.seg[v], hi = tab.seg[v + 1];
    const uint64_t target = (uint64_t)b * block_rows;
    while (lo < hi) {
        uint32_t mid = lo + ((hi - lo) >> 1);
        if ((uint64_t)sig_o[mid] < target) lo = mid + 1;
        else hi = mid;
    }
    bounds[t] = lo;
}

}  // namespace
}  // namespace fgx
