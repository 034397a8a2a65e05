// Times LlamaContextDecoder<half> -- the whole stack of prefill layers -- at the LLaMA-2-7B shape with dummy
// weights and prints one JSON line.
//   bench_context_decoder <layers> <iterations> <warmup> <max_q_len> <len_0> <len_1> ...
// One iteration = one forward() over the ragged batch (history 0): padding offsets, the first RMSNorm and
// `layers` decoder layers, HIP events on the null stream around all iterations.  Used by bench.py for its
// `context_decoder_cpp` record.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <numeric>
#include <vector>

#include "src/layers/decoder/context_decoder.h"
#include "src/memory/allocator/hip_allocator.h"

template <typename V>
static V* upload(const std::vector<V>& h) {
    V* d = nullptr;
    CHECK(hipMalloc((void**)&d, h.size() * sizeof(V) + 16));
    CHECK(hipMemcpy(d, h.data(), h.size() * sizeof(V), hipMemcpyHostToDevice));
    return d;
}

int main(int argc, char** argv) {
    if (argc < 6) {
        std::printf("usage: bench_context_decoder <layers> <iterations> <warmup> <max_q_len> <len_0> ...\n");
        return 2;
    }
    const int layers = std::atoi(argv[1]), iterations = std::atoi(argv[2]), warmup = std::atoi(argv[3]);
    const int max_q = std::atoi(argv[4]);
    std::vector<int> lens;
    for (int i = 5; i < argc; i++) lens.push_back(std::atoi(argv[i]));
    const int batch = (int)lens.size(), tokens = std::accumulate(lens.begin(), lens.end(), 0);
    const int head_num = 32, kv_heads = 32, head_size = 128, inter = 11008, hidden = head_num * head_size;
    const int max_k = *std::max_element(lens.begin(), lens.end());
    try {
        HipAllocator allocator;
        LLaMAAttentionStaticParams params;
        std::vector<std::unique_ptr<LlamaLayerWeight<half>>> owned;
        std::vector<LlamaLayerWeight<half>*> weights;
        for (int l = 0; l < layers; l++) {
            owned.emplace_back(new LlamaLayerWeight<half>(head_num, kv_heads, head_size, inter, WeightType::FP16_W, false));
            owned.back()->loadWeights();
            weights.push_back(owned.back().get());
        }
        LlamaContextDecoder<half> decoder(head_num, kv_heads, head_size, inter, layers, params, 1e-5f, &allocator);
        std::vector<half> rows((size_t)tokens * hidden);
        for (size_t i = 0; i < rows.size(); i++) rows[i] = __float2half((float)((i * 2654435761u >> 16) & 1023) / 512.0f - 1.0f);
        half* embedded = upload(rows);
        half* out = upload(rows);
        const size_t cache_elems = (size_t)layers * batch * kv_heads * max_q * head_size;
        half *k_cache = nullptr, *v_cache = nullptr;
        CHECK(hipMalloc((void**)&k_cache, cache_elems * sizeof(half)));
        CHECK(hipMalloc((void**)&v_cache, cache_elems * sizeof(half)));
        CHECK(hipMemset(k_cache, 0, cache_elems * sizeof(half)));
        CHECK(hipMemset(v_cache, 0, cache_elems * sizeof(half)));
        int* d_lens = upload(lens);
        int* d_hist = upload(std::vector<int>(batch, 0));
        const DataType dt = getTensorType<half>();
        TensorWrapper<int> il(Device::GPU, getTensorType<int>(), {batch}, d_lens);
        TensorWrapper<int> hl(Device::GPU, getTensorType<int>(), {batch}, d_hist);
        TensorWrapper<half> in(Device::GPU, dt, {tokens, hidden}, embedded);
        TensorWrapper<half> o(Device::GPU, dt, {tokens, hidden}, out);
        TensorWrapper<half> kc(Device::GPU, dt, {layers, batch, kv_heads, max_q, head_size}, k_cache);
        TensorWrapper<half> vc(Device::GPU, dt, {layers, batch, kv_heads, max_q, head_size}, v_cache);
        TensorMap inputs{{"decoder_input", &in}, {"history_length", &hl}, {"input_length", &il}, {"context_length", &il}};
        TensorMap outputs{{"decoder_output", &o}, {"all_k_cache", &kc}, {"all_v_cache", &vc}};
        LLaMAAttentionDynParams dyn;
        dyn.batch_size = batch, dyn.num_tokens = tokens, dyn.max_q_len = max_q, dyn.max_k_len = max_k, dyn.num_layers = layers;
        for (int i = 0; i < warmup; i++) decoder.forward(inputs, weights, weights[0]->ffn_norm_weight, outputs, dyn);
        CHECK(hipDeviceSynchronize());
        hipEvent_t e0, e1;
        CHECK(hipEventCreate(&e0));
        CHECK(hipEventCreate(&e1));
        CHECK(hipEventRecord(e0, nullptr));
        for (int i = 0; i < iterations; i++) decoder.forward(inputs, weights, weights[0]->ffn_norm_weight, outputs, dyn);
        CHECK(hipEventRecord(e1, nullptr));
        CHECK(hipEventSynchronize(e1));
        float ms = 0.f;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        ms /= (float)iterations;
        std::printf("{\"workload\": \"llama2_7b_context_decoder_f16_cpp\", \"layers\": %d, \"valid_tokens\": %d, \"batch\": %d, "
                    "\"max_q_len\": %d, \"ms_per_forward\": %.4f, \"ms_per_layer\": %.4f, \"prefill_tokens_per_s\": %.1f, "
                    "\"iterations\": %d, "
                    "\"note\": \"C++ LlamaContextDecoder: padding offsets + first RMSNorm + the layer stack (launch* kernels, "
                    "hipBLASLt GEMMs, attention fused on the matrix cores unless ISP_LAYERS_ATTENTION=padded); embedding and LM head excluded\"}\n",
                    layers, tokens, batch, max_q, ms, ms / layers, tokens / (ms * 1e-3), iterations);
    } catch (const std::exception& e) {
        std::printf("exception: %s\n", e.what());
        return 1;
    }
    return 0;
}
