// Times the context layer's fused attention kernel alone at the LLaMA-2-7B layer shape and prints one JSON line.
//   bench_context_attention <iterations> <warmup> <max_q_len> <len_0> <len_1> ...
// 32 query heads and 32 key heads of 128 elements, history 0, random fp16 operands.  Reported: microseconds per
// launch (HIP events on the null stream around all iterations); the matrix-core rate over the flops the causal
// mask leaves (4 * head_size flops per visible (query, key) pair) against the 2.5 PFLOP/s fp16 peak; and the bytes
// the kernel cannot avoid (queries and results once, each sequence's keys and values once) against 8 TB/s.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <numeric>
#include <random>
#include <vector>

#include "src/layers/decoder/context_decoder_layer.h"
#include "src/utils/macro.h"

template <typename V>
static V* upload(const std::vector<V>& h) {
    V* d = nullptr;
    CHECK(hipMalloc((void**)&d, h.size() * sizeof(V) + 16));
    CHECK(hipMemcpy(d, h.data(), h.size() * sizeof(V), hipMemcpyHostToDevice));
    return d;
}

int main(int argc, char** argv) {
    if (argc < 5) {
        std::printf("usage: bench_context_attention <iterations> <warmup> <max_q_len> <len_0> ...\n");
        return 2;
    }
    const int iterations = std::atoi(argv[1]), warmup = std::atoi(argv[2]), max_q = std::atoi(argv[3]);
    std::vector<int> lens;
    for (int i = 4; i < argc; i++) lens.push_back(std::atoi(argv[i]));
    const int batch = (int)lens.size(), tokens = std::accumulate(lens.begin(), lens.end(), 0);
    const int heads = 32, kv_heads = 32, hs = 128, max_seq = max_q;
    try {
        std::mt19937 gen(1);
        std::normal_distribution<float> dist(0.f, 1.f);
        std::vector<half> q((size_t)batch * heads * max_q * hs), k((size_t)batch * kv_heads * max_seq * hs), v(k.size());
        for (auto& x : q) x = __float2half(dist(gen));
        for (auto& x : k) x = __float2half(dist(gen));
        for (auto& x : v) x = __float2half(dist(gen));
        half *dq = upload(q), *dk = upload(k), *dv = upload(v), *dout = upload(std::vector<half>((size_t)tokens * heads * hs));
        int *dl = upload(lens), *dh = upload(std::vector<int>(batch, 0));
        auto launch = [&] {
            isp_layers::launch_fused_context_attention(dq, dk, dv, dout, dh, dl, dl, batch, heads, kv_heads, hs, max_q, max_q,
                                                       max_seq, tokens, 1.0f / std::sqrt((float)hs));
        };
        for (int i = 0; i < warmup; i++) launch();
        hipEvent_t e0, e1;
        CHECK(hipEventCreate(&e0));
        CHECK(hipEventCreate(&e1));
        CHECK(hipEventRecord(e0, nullptr));
        for (int i = 0; i < iterations; i++) launch();
        CHECK(hipEventRecord(e1, nullptr));
        CHECK(hipEventSynchronize(e1));
        float ms = 0.f;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        const double us = ms * 1e3 / iterations;
        double pairs = 0, kv_rows = 0;
        for (int l : lens) pairs += 0.5 * l * (l + 1.0), kv_rows += l;
        const double flops = 4.0 * hs * pairs * heads;
        const double floor_bytes = 2.0 * tokens * heads * hs * 2 + 2.0 * kv_rows * kv_heads * hs * 2;
        std::printf("{\"workload\": \"fused_context_attention_f16_b%d_s%d_h%dx%d\", \"valid_tokens\": %d, \"us_per_launch\": %.2f, "
                    "\"causal_flops\": %.0f, \"TFLOPs\": %.1f, \"frac_of_fp16_mfma_peak\": %.3f, \"unavoidable_bytes\": %.0f, "
                    "\"us_at_8TBs\": %.2f, \"iterations\": %d}\n",
                    batch, max_q, heads, hs, tokens, us, flops, flops / us * 1e-6, flops / us * 1e-6 / 2500.0, floor_bytes,
                    floor_bytes / 8e6, iterations);
    } catch (const std::exception& e) {
        std::printf("exception: %s\n", e.what());
        return 1;
    }
    return 0;
}
