// The neighbor cache of a submanifold convolution in one call: the map and its mask codes (sort-and-merge builder), the
// mask sort, and for a training cache the pair lists -- the calls a host would otherwise make one after the other, each
// with its allocations and argument marshalling in between while the GPU waits.  The pair lists and the mask sort both
// start from the map and need nothing of each other; from a few hundred thousand voxels on the lists are enqueued on a
// second stream of the library's own (default priority, one per device, made on first use), which the caller's stream
// waits for before the call returns.
#include <mutex>

#include "fgx_common.h"

namespace fgx {
namespace {

constexpr int kMaxCacheDevices = 64;
constexpr size_t kTwoStreamsMinRows = 393216;      // below, the second stream's events cost more than the overlap gives

hipStream_t g_side_stream[kMaxCacheDevices];
std::mutex g_side_mutex;

int side_stream(hipStream_t* out) {
    int dev = 0;
    FGX_CHECK_HIP(hipGetDevice(&dev));
    FGX_CHECK_ARG(dev >= 0 && dev < kMaxCacheDevices, "fgx_subm_cache_build: device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_side_mutex);
    if (g_side_stream[dev] == nullptr) FGX_CHECK_HIP(hipStreamCreateWithFlags(&g_side_stream[dev], hipStreamNonBlocking));
    *out = g_side_stream[dev];
    return FGX_OK;
}

struct CacheLayout {
    size_t map_ws, map_bytes, sort_ws, sort_bytes, pair_ws, pair_bytes, total;
};

CacheLayout cache_layout(size_t n, int key_bits, int Kw, int Kh, int V, int with_pairs) {
    CacheLayout L{};
    L.map_bytes = fgx_subm_neighbor_map_sorted_workspace_bytes(n, key_bits, Kw, Kh);
    L.sort_bytes = fgx_sort_workspace_bytes(n);
    L.pair_bytes = with_pairs ? fgx_pair_workspace_bytes(n, V) : 0;
    size_t off = 0;
    L.map_ws = off;
    off = align_up(off + L.map_bytes, 256);
    L.sort_ws = off;
    off = align_up(off + L.sort_bytes, 256);
    L.pair_ws = off;
    off = align_up(off + L.pair_bytes, 256);
    L.total = off;
    return L;
}

}  // namespace
}  // namespace fgx

using namespace fgx;

extern "C" size_t fgx_subm_cache_workspace_bytes(size_t n, int key_bits, int Kw, int Kh, int Kd, int with_pairs) {
    if ((key_bits != 32 && key_bits != 64) || Kw < 1 || Kh < 1 || Kd < 1 || (long long)Kw * Kh * Kd > 32) return 0;
    if (fgx_subm_neighbor_map_sorted_workspace_bytes(n, key_bits, Kw, Kh) == 0) return 0;
    return cache_layout(n, key_bits, Kw, Kh, Kw * Kh * Kd, with_pairs).total;
}

extern "C" int fgx_subm_cache_build(const int32_t* coords, size_t n, int B, int W, int H, int D, int Kw, int Kh, int Kd, int Dw,
                                    int Dh, int Dd, int key_bits, int presorted, int with_pairs, void* workspace,
                                    size_t workspace_bytes, uint32_t* out_map, int32_t* gray, int32_t* binary,
                                    int64_t* sorted_idx, uint32_t* seg, uint32_t* sig_i, uint32_t* sig_o, fgx_stream_t stream) {
    FGX_CHECK_ARG(Kw > 0 && Kh > 0 && Kd > 0 && (long long)Kw * Kh * Kd <= 32,
                  "fgx_subm_cache_build: mask codes need a kernel volume <= 32, got (%d,%d,%d)", Kw, Kh, Kd);
    const int V = Kw * Kh * Kd;
    FGX_CHECK_ARG(!with_pairs || seg != nullptr, "fgx_subm_cache_build: null segment table");
    FGX_CHECK_ARG(n * (size_t)V < 0xFFFFFFFFull, "fgx_subm_cache_build: pair offsets must fit in 32 bits");
    hipStream_t s = (hipStream_t)stream;
    if (n == 0) return with_pairs ? fgx_pair_count(nullptr, 0, V, seg, nullptr, 0, stream) : FGX_OK;
    FGX_CHECK_ARG(key_bits == 32 || key_bits == 64, "fgx_subm_cache_build: key_bits must be 32 or 64, got %d", key_bits);
    FGX_CHECK_ARG(coords && workspace && out_map && gray && binary && sorted_idx, "fgx_subm_cache_build: null buffer");
    FGX_CHECK_ARG(!with_pairs || (sig_i && sig_o), "fgx_subm_cache_build: null pair list");
    FGX_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "fgx_subm_cache_build: workspace must be 256-byte aligned");
    const CacheLayout L = cache_layout(n, key_bits, Kw, Kh, V, with_pairs);
    FGX_CHECK_ARG(L.map_bytes != 0, "fgx_subm_cache_build: kernel of %d x %d rows is too large for the sorted builder", Kw, Kh);
    FGX_CHECK_ARG(workspace_bytes >= L.total, "fgx_subm_cache_build: workspace of %zu bytes, need %zu", workspace_bytes, L.total);
    char* ws = (char*)workspace;

    int rc = fgx_subm_neighbor_map_sorted(coords, n, B, W, H, D, Kw, Kh, Kd, Dw, Dh, Dd, key_bits, presorted, ws + L.map_ws,
                                          L.map_bytes, out_map, gray, binary, stream);
    if (rc != FGX_OK) return rc;

    // a second stream only outside a capture (a capture would have to own it) and where it pays
    bool two_streams = with_pairs && n >= kTwoStreamsMinRows;
    if (two_streams) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        FGX_CHECK_HIP(hipStreamIsCapturing(s, &capturing));
        two_streams = capturing == hipStreamCaptureStatusNone;
    }
    hipStream_t side = nullptr;
    hipEvent_t map_made = nullptr, lists_made = nullptr;
    if (two_streams) {
        rc = side_stream(&side);
        if (rc != FGX_OK) return rc;
        FGX_CHECK_HIP(hipEventCreateWithFlags(&map_made, hipEventDisableTiming));
        hipError_t e = hipEventCreateWithFlags(&lists_made, hipEventDisableTiming);
        if (e == hipSuccess) e = hipEventRecord(map_made, s);
        if (e != hipSuccess) {
            (void)hipEventDestroy(map_made);
            if (lists_made) (void)hipEventDestroy(lists_made);
            return fail_hip(e, "fgx_subm_cache_build(events)");
        }
    }
    // the mask sort first: it is the longer of the two chains
    rc = fgx_sort_by_code(binary, n, V, sorted_idx, ws + L.sort_ws, L.sort_bytes, stream);
    if (rc == FGX_OK && with_pairs) {
        const fgx_stream_t lists_on = two_streams ? (fgx_stream_t)side : stream;
        hipError_t e = two_streams ? hipStreamWaitEvent(side, map_made, 0) : hipSuccess;
        if (e != hipSuccess) rc = fail_hip(e, "fgx_subm_cache_build(wait for the map)");
        if (rc == FGX_OK) rc = fgx_pair_count(gray, n, V, seg, ws + L.pair_ws, L.pair_bytes, lists_on);
        if (rc == FGX_OK) rc = fgx_pair_fill(out_map, gray, n, V, ws + L.pair_ws, sig_i, sig_o, lists_on);
        if (two_streams) {
            // whatever was enqueued on the second stream, the caller's stream waits for it: its buffers are the caller's
            e = hipEventRecord(lists_made, side);
            if (e == hipSuccess) e = hipStreamWaitEvent(s, lists_made, 0);
            if (e != hipSuccess && rc == FGX_OK) rc = fail_hip(e, "fgx_subm_cache_build(join)");
        }
    }
    if (map_made) (void)hipEventDestroy(map_made);
    if (lists_made) (void)hipEventDestroy(lists_made);
    return rc;
}
