// Shared helpers of the gfx950 kernels behind the C ABI declared in include/flexgemm_hip.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <stdio.h>

#include "../../include/flexgemm_hip.h"

#define FGX_EMPTY32 0xFFFFFFFFu

namespace fgx {

// Thread-local message behind fgx_last_error().
void set_error(const char* fmt, ...);

inline int fail_hip(hipError_t e, const char* what) {
    set_error("%s: %s", what, hipGetErrorString(e));
    return FGX_ERR_HIP;
}

#define FGX_CHECK_ARG(cond, ...)                 \
    do {                                         \
        if (!(cond)) {                           \
            ::fgx::set_error(__VA_ARGS__);       \
            return FGX_ERR_ARG;                  \
        }                                        \
    } while (0)

#define FGX_CHECK_LAUNCH(what)                                   \
    do {                                                         \
        hipError_t e_ = hipGetLastError();                       \
        if (e_ != hipSuccess) return ::fgx::fail_hip(e_, what);  \
    } while (0)

#define FGX_CHECK_HIP(expr)                                      \
    do {                                                         \
        hipError_t e_ = (expr);                                  \
        if (e_ != hipSuccess) return ::fgx::fail_hip(e_, #expr); \
    } while (0)

// Names the phase whose kernels are enqueued next on `s` to the profiling hook (fgx_set_phase_hook), if one is set;
// an empty name closes the last phase of a call.
void phase_mark(const char* name, hipStream_t s);
// closes the last phase when the call returns, by whichever path
struct PhaseEnd {
    hipStream_t s;
    ~PhaseEnd() { phase_mark("", s); }
};

// Whether the persistent gather GEMM of this tile shape has room in a CU's 160 KiB of LDS for `cols` output columns
// (it stages the bias of every column tile next to its rings); defined in conv_gemm_stream.hip.
bool stream_lds_fits(int tile_rows, int tile_cols, int slab_bytes, int cols);

inline unsigned cdiv(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

}  // namespace fgx
