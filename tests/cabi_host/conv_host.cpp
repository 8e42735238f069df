// A caller of the C ABI with no Python and no torch in the process: plain HIP host calls for memory, the library's entry
// points for everything else.  One submanifold 3x3x3 convolution in fp32 on a random half-filled grid -- neighbor cache in
// one call, forward, input gradient, weight and bias gradient -- checked against loops on the host written from the
// definition of the operator (flex_gemm/ops/spconv/submanifold_conv3d.py:109-168 of the reference is the same
// arithmetic through an explicit im2col).  Prints "ok" and exits 0, or says what differs and exits 1.
//
// Test infrastructure: built next to the library and run by the GPU tests; nothing in the product uses it.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <tuple>
#include <vector>

#include "flexgemm_hip.h"

#define HIP_OK(call)                                                                                   \
    do {                                                                                               \
        hipError_t e_ = (call);                                                                        \
        if (e_ != hipSuccess) {                                                                        \
            std::fprintf(stderr, "%s: %s (line %d)\n", #call, hipGetErrorString(e_), __LINE__);        \
            std::exit(1);                                                                              \
        }                                                                                              \
    } while (0)
#define FGX(call)                                                                                      \
    do {                                                                                               \
        if ((call) != FGX_OK) {                                                                        \
            std::fprintf(stderr, "%s: %s (line %d)\n", #call, fgx_last_error(), __LINE__);             \
            std::exit(1);                                                                              \
        }                                                                                              \
    } while (0)

namespace {

template <typename T>
T* device(size_t count) {
    void* p = nullptr;
    HIP_OK(hipMalloc(&p, (count ? count : 1) * sizeof(T)));
    return (T*)p;
}
void* device_bytes(size_t bytes) {
    void* p = nullptr;
    HIP_OK(hipMalloc(&p, bytes ? bytes : 256));
    return p;
}
template <typename T>
T* upload(const std::vector<T>& h) {
    T* d = device<T>(h.size());
    HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
}
template <typename T>
std::vector<T> download(const T* d, size_t count) {
    std::vector<T> h(count);
    HIP_OK(hipMemcpy(h.data(), d, count * sizeof(T), hipMemcpyDeviceToHost));
    return h;
}

uint32_t lcg_state = 12345u;
float uniform() {      // (-1, 1)
    lcg_state = lcg_state * 1664525u + 1013904223u;
    return ((lcg_state >> 8) * (1.0f / 8388608.0f)) - 1.0f;
}

double worst(const std::vector<float>& got, const std::vector<double>& ref) {
    double peak = 0, err = 0;
    for (size_t i = 0; i < ref.size(); ++i) {
        peak = std::fmax(peak, std::fabs(ref[i]));
        err = std::fmax(err, std::fabs((double)got[i] - ref[i]));
    }
    return err / (peak > 0 ? peak : 1);
}

}  // namespace

int main(int argc, char** argv) {
    const int res = argc > 1 ? std::atoi(argv[1]) : 14, Ci = argc > 2 ? std::atoi(argv[2]) : 24, Co = argc > 3 ? std::atoi(argv[3]) : 40;
    const int V = 27;
    std::printf("conv_host: grid %d^3, Ci=%d Co=%d fp32\n", res, Ci, Co);
    std::fflush(stdout);

    // every second cell of the grid, in a shuffled order
    std::vector<int32_t> coords;
    for (int x = 0; x < res; ++x)
        for (int y = 0; y < res; ++y)
            for (int z = 0; z < res; ++z)
                if (uniform() > 0.f) coords.insert(coords.end(), {0, x, y, z});
    size_t n = coords.size() / 4;
    for (size_t i = n - 1; i > 0; --i) {
        lcg_state = lcg_state * 1664525u + 1013904223u;
        const size_t j = (lcg_state >> 4) % (i + 1);
        for (int c = 0; c < 4; ++c) std::swap(coords[4 * i + c], coords[4 * j + c]);
    }
    std::map<std::tuple<int, int, int>, uint32_t> row_of;
    for (size_t i = 0; i < n; ++i) row_of[{coords[4 * i + 1], coords[4 * i + 2], coords[4 * i + 3]}] = (uint32_t)i;
    // the operator's definition of the map: offset v = ((dx + 1) * 3 + dy + 1) * 3 + dz + 1, absent = all ones
    std::vector<uint32_t> map_ref(n * V, 0xFFFFFFFFu);
    for (size_t i = 0; i < n; ++i)
        for (int v = 0; v < V; ++v) {
            const int dx = v / 9 - 1, dy = v / 3 % 3 - 1, dz = v % 3 - 1;
            auto it = row_of.find({coords[4 * i + 1] + dx, coords[4 * i + 2] + dy, coords[4 * i + 3] + dz});
            if (it != row_of.end()) map_ref[i * V + v] = it->second;
        }
    std::vector<float> feats(n * Ci), weight((size_t)Co * V * Ci), bias(Co), grad(n * Co);
    for (auto& x : feats) x = uniform();
    for (auto& x : weight) x = uniform() / std::sqrt((float)(V * Ci));
    for (auto& x : bias) x = uniform();
    for (auto& x : grad) x = uniform();

    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    int32_t* d_coords = upload(coords);
    float *d_feats = upload(feats), *d_weight = upload(weight), *d_bias = upload(bias), *d_grad = upload(grad);

    // ---- neighbor cache in one call
    uint32_t* d_map = device<uint32_t>(n * V);
    int32_t *d_gray = device<int32_t>(n), *d_binary = device<int32_t>(n);
    int64_t* d_sorted = device<int64_t>(n);
    uint32_t *d_seg = device<uint32_t>(V + 1), *d_sig_i = device<uint32_t>(n * V), *d_sig_o = device<uint32_t>(n * V);
    const size_t cache_ws_bytes = fgx_subm_cache_workspace_bytes(n, 32, 3, 3, 3, 1);
    if (cache_ws_bytes == 0) {
        std::fprintf(stderr, "fgx_subm_cache_workspace_bytes said 0\n");
        return 1;
    }
    void* cache_ws = device_bytes(cache_ws_bytes);
    FGX(fgx_subm_cache_build(d_coords, n, 1, res, res, res, 3, 3, 3, 1, 1, 1, 32, 0, 1, cache_ws, cache_ws_bytes, d_map, d_gray,
                             d_binary, d_sorted, d_seg, d_sig_i, d_sig_o, stream));
    HIP_OK(hipStreamSynchronize(stream));
    if (download(d_map, n * V) != map_ref) {
        std::fprintf(stderr, "neighbor map differs from the definition\n");
        return 1;
    }
    std::vector<uint32_t> seg = download(d_seg, V + 1);
    size_t pairs_ref = 0;
    for (uint32_t m : map_ref) pairs_ref += m != 0xFFFFFFFFu;
    if (seg[V] != pairs_ref) {
        std::fprintf(stderr, "pair count %u, expected %zu\n", seg[V], pairs_ref);
        return 1;
    }
    std::printf("  cache: %zu voxels, %zu pairs\n", n, pairs_ref);
    std::fflush(stdout);

    // ---- forward (pass 0) and input gradient (pass 1) on the tiled gather GEMM
    float *d_out = device<float>(n * Co), *d_gi = device<float>(n * Ci);
    for (int pass = 0; pass < 2; ++pass) {
        fgx_schedule sch;
        FGX(fgx_table_lookup(pass, FGX_F32, n, Ci, Co, V, &sch));
        const size_t tiles = (n + sch.tile_rows - 1) / sch.tile_rows;
        int32_t *d_tile_code = device<int32_t>(tiles), *d_tile_seg = device<int32_t>(tiles + 1);
        const size_t tile_ws_bytes = fgx_tile_workspace_bytes(n, sch.tile_rows);
        void* tile_ws = device_bytes(tile_ws_bytes);
        FGX(fgx_tile_codes(d_gray, d_sorted, n, sch.tile_rows, d_tile_code, d_tile_seg, tile_ws, tile_ws_bytes, stream));
        const size_t panel_bytes = fgx_weight_panel_bytes(FGX_F32, pass, Ci, Co, V, sch.slab_bytes, sch.tile_cols);
        void* panel = device_bytes(panel_bytes);
        FGX(fgx_pack_weight(FGX_F32, pass, d_weight, Ci, Co, V, sch.slab_bytes, sch.tile_cols, panel, stream));
        const int K = pass == 0 ? Ci : Co, cols = pass == 0 ? Co : Ci;
        void* scratch = sch.splitk > 1 ? device_bytes(fgx_conv_scratch_bytes(n, cols, sch.splitk)) : nullptr;
        FGX(fgx_conv_gather_gemm(FGX_F32, pass == 0 ? d_feats : d_grad, panel, pass == 0 ? d_bias : nullptr, d_map, d_sorted,
                                 d_tile_code, n, K, cols, V, sch.tile_rows, sch.tile_cols, sch.slab_bytes, sch.splitk, scratch,
                                 pass == 0 ? d_out : d_gi, stream));
        HIP_OK(hipStreamSynchronize(stream));
        HIP_OK(hipFree(d_tile_code));
        HIP_OK(hipFree(d_tile_seg));
        HIP_OK(hipFree(tile_ws));
        HIP_OK(hipFree(panel));
        if (scratch) HIP_OK(hipFree(scratch));
    }

    // ---- weight and bias gradient
    fgx_schedule sch;
    FGX(fgx_table_lookup(2, FGX_F32, n, Ci, Co, V, &sch));
    void* wgrad_scratch = device_bytes(fgx_wgrad_scratch_bytes(n, V, Ci, Co, sch.block_rows));
    float *d_gw = device<float>((size_t)Co * V * Ci), *d_gb = device<float>(Co);
    FGX(fgx_conv_wgrad(FGX_F32, d_grad, d_feats, d_sig_i, d_sig_o, seg.data(), nullptr, n, n, Ci, Co, V, sch.tile_rows,
                       sch.tile_cols, sch.block_rows, sch.stream == 1, wgrad_scratch, d_gw, d_gb, 13, stream));
    HIP_OK(hipStreamSynchronize(stream));

    // ---- the same four results from the definition, in double
    std::vector<double> out_ref(n * Co), gi_ref(n * Ci, 0.0), gw_ref((size_t)Co * V * Ci, 0.0), gb_ref(Co, 0.0);
    for (size_t i = 0; i < n; ++i) {
        for (int o = 0; o < Co; ++o) {
            out_ref[i * Co + o] = bias[o];
            gb_ref[o] += grad[i * Co + o];
        }
        for (int v = 0; v < V; ++v) {
            const uint32_t j = map_ref[i * V + v];
            if (j == 0xFFFFFFFFu) continue;
            for (int o = 0; o < Co; ++o) {
                const float* w = &weight[((size_t)o * V + v) * Ci];
                const double g = grad[i * Co + o];
                double s = 0;
                for (int c = 0; c < Ci; ++c) {
                    s += (double)w[c] * feats[(size_t)j * Ci + c];
                    gi_ref[(size_t)j * Ci + c] += g * w[c];
                    gw_ref[((size_t)o * V + v) * Ci + c] += g * feats[(size_t)j * Ci + c];
                }
                out_ref[i * Co + o] += s;
            }
        }
    }
    const double e_out = worst(download(d_out, n * Co), out_ref), e_gi = worst(download(d_gi, n * Ci), gi_ref);
    const double e_gw = worst(download(d_gw, (size_t)Co * V * Ci), gw_ref), e_gb = worst(download(d_gb, Co), gb_ref);
    std::printf("  max error / max value: forward %.2e, input gradient %.2e, weight gradient %.2e, bias gradient %.2e\n", e_out,
                e_gi, e_gw, e_gb);
    const double tol = 1e-4;        // fp32 inputs: the tolerance of the Python suite
    if (!(e_out < tol && e_gi < tol && e_gw < tol && e_gb < tol)) {
        std::fprintf(stderr, "a result is off by more than %.0e\n", tol);
        return 1;
    }
    HIP_OK(hipStreamDestroy(stream));
    std::printf("ok\n");
    return 0;
}
