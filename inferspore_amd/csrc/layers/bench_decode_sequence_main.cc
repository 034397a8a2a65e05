// What a decode step's worth of this library's kernels costs a C++ caller: the five launch-bound kernels of a
// step for a batch of 16 (fused norm, fused bias + RoPE + KV append, KV broadcast, SwiGLU, RMSNorm) issued
// back to back through the C ABI on one stream, and the same sequence replayed from a captured HIP graph.
// Prints one JSON line; bench.py merges it into its `decode_sequence` record (whose own figures are taken
// from Python, where each launch costs a ctypes call).
//   bench_decode_sequence <steps>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#include "inferspore_amd.h"

#define HIP_OK(call)                                                                   \
    do {                                                                               \
        const hipError_t e_ = (call);                                                  \
        if (e_ != hipSuccess) {                                                        \
            std::printf("%s failed: %s\n", #call, hipGetErrorString(e_));              \
            return 1;                                                                  \
        }                                                                              \
    } while (0)

template <typename V>
static V* device_filled(size_t n, float value) {
    std::vector<V> h(n);
    for (size_t i = 0; i < n; i++) h[i] = (V)(value * (float)((i * 2654435761u >> 20) & 255) / 255.0f);
    V* d = nullptr;
    if (hipMalloc((void**)&d, n * sizeof(V)) != hipSuccess) return nullptr;
    if (hipMemcpy(d, h.data(), n * sizeof(V), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
    return d;
}

int main(int argc, char** argv) {
    const int steps = argc > 1 ? std::atoi(argv[1]) : 500;
    const int batch = 16, heads = 32, kv_heads = 32, hs = 128, hidden = 4096, inter = 11008, max_seq = 256, ctx_len = 101;
    if (isp_init() != ISP_OK) {
        std::printf("no gfx950 device\n");
        return 1;
    }
    half* hidden_rows = device_filled<half>((size_t)batch * hidden, 1.0f);
    half* residual = device_filled<half>((size_t)batch * hidden, 1.0f);
    half* gamma = device_filled<half>(hidden, 1.0f);
    half* qkv = device_filled<half>((size_t)batch * (heads + 2 * kv_heads) * hs, 1.0f);
    half* k_cache = device_filled<half>((size_t)batch * kv_heads * max_seq * hs, 1.0f);
    half* v_cache = device_filled<half>((size_t)batch * kv_heads * max_seq * hs, 1.0f);
    half* k_rep = device_filled<half>((size_t)batch * heads * ctx_len * hs, 0.0f);
    half* v_rep = device_filled<half>((size_t)batch * heads * ctx_len * hs, 0.0f);
    half* gate_up = device_filled<half>((size_t)batch * 2 * inter, 1.0f);
    half* act_out = device_filled<half>((size_t)batch * inter, 0.0f);
    std::vector<int> h_hist(batch, ctx_len - 1), h_ctx(batch, ctx_len);
    int *hist = nullptr, *ctx = nullptr;
    HIP_OK(hipMalloc((void**)&hist, batch * sizeof(int)));
    HIP_OK(hipMalloc((void**)&ctx, batch * sizeof(int)));
    HIP_OK(hipMemcpy(hist, h_hist.data(), batch * sizeof(int), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(ctx, h_ctx.data(), batch * sizeof(int), hipMemcpyHostToDevice));
    if (!hidden_rows || !residual || !gamma || !qkv || !k_cache || !v_cache || !k_rep || !v_rep || !gate_up || !act_out) {
        std::printf("allocation failed\n");
        return 1;
    }
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    int failed = 0;
    auto step = [&] {
        failed |= isp_fused_add_bias_residual_rmsnorm_f16(residual, hidden_rows, nullptr, gamma, 1e-5f, batch, hidden, 0u, stream);
        failed |= isp_rope_decode_append_f16(qkv, nullptr, k_cache, v_cache, 0, max_seq, hist, batch, heads, kv_heads, hs,
                                             ctx_len, hs, 10000.0f, stream);
        failed |= isp_repeat_kv_cache_f16(k_cache, v_cache, k_rep, v_rep, 0, ctx, batch, heads, kv_heads, max_seq, ctx_len, hs,
                                          stream);
        failed |= isp_swiglu_f16(gate_up, act_out, batch, inter, stream);
        failed |= isp_rmsnorm_f16(hidden_rows, gamma, 1e-5f, batch, hidden, stream);
    };
    hipEvent_t e0, e1;
    HIP_OK(hipEventCreate(&e0));
    HIP_OK(hipEventCreate(&e1));
    for (int i = 0; i < 20; i++) step();
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipEventRecord(e0, stream));
    for (int i = 0; i < steps; i++) step();
    HIP_OK(hipEventRecord(e1, stream));
    HIP_OK(hipEventSynchronize(e1));
    float eager_ms = 0.f;
    HIP_OK(hipEventElapsedTime(&eager_ms, e0, e1));

    hipGraph_t graph;
    hipGraphExec_t exec;
    HIP_OK(hipStreamBeginCapture(stream, hipStreamCaptureModeThreadLocal));
    step();
    HIP_OK(hipStreamEndCapture(stream, &graph));
    HIP_OK(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0));
    for (int i = 0; i < 20; i++) HIP_OK(hipGraphLaunch(exec, stream));
    HIP_OK(hipStreamSynchronize(stream));
    HIP_OK(hipEventRecord(e0, stream));
    for (int i = 0; i < steps; i++) HIP_OK(hipGraphLaunch(exec, stream));
    HIP_OK(hipEventRecord(e1, stream));
    HIP_OK(hipEventSynchronize(e1));
    float graph_ms = 0.f;
    HIP_OK(hipEventElapsedTime(&graph_ms, e0, e1));
    if (failed) {
        std::printf("a launch failed: %s (hip %d)\n", isp_strerror(ISP_ERR_LAUNCH), isp_last_hip_error());
        return 1;
    }
    std::printf("{\"cpp_fused_eager_us_per_step\": %.2f, \"cpp_fused_graph_replay_us_per_step\": %.2f, "
                "\"cpp_steps\": %d, \"cpp_kernels_per_step\": 5}\n",
                eager_ms * 1e3 / steps, graph_ms * 1e3 / steps, steps);
    return 0;
}
