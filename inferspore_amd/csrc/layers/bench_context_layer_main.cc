// Times LlamaContextDecoderLayer<half> at a LLaMA-2-7B shape with dummy weights and prints one JSON line.
//   bench_context_layer [--history H] <iterations> <warmup> <max_q_len> <len_0> <len_1> ...
// One iteration = one forward() of one layer over the whole ragged batch (every sequence with H tokens already in
// the KV cache, 0 by default; H > 0 with max_q_len = 1 is a decode step), HIP events on the null stream around
// all iterations.  Used by bench.py for its `context_layer_cpp` record.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <vector>

#include "src/kernels/cal_paddingoffset.h"
#include "src/layers/decoder/context_decoder_layer.h"
#include "src/memory/allocator/hip_allocator.h"

template <typename V>
static V* upload(const std::vector<V>& h) {
    V* d = nullptr;
    CHECK(hipMalloc((void**)&d, h.size() * sizeof(V) + 16));
    CHECK(hipMemcpy(d, h.data(), h.size() * sizeof(V), hipMemcpyHostToDevice));
    return d;
}

static const char* attention_kind() {
    const char* a = std::getenv("ISP_LAYERS_ATTENTION");
    return a != nullptr && std::strcmp(a, "padded") == 0 ? "padded" : "fused";
}

int main(int argc, char** argv) {
    // --history H: every sequence already has H tokens in the KV cache (a later turn, or with max_q_len = 1 and
    // lengths of 1 a decode step)
    int history = 0;
    if (argc > 2 && std::strcmp(argv[1], "--history") == 0) {
        history = std::atoi(argv[2]);
        argv += 2;
        argc -= 2;
    }
    if (argc < 5 || history < 0) {
        std::printf("usage: bench_context_layer [--history H] <iterations> <warmup> <max_q_len> <len_0> ...\n");
        return 2;
    }
    const int iterations = std::atoi(argv[1]), warmup = std::atoi(argv[2]), max_q = std::atoi(argv[3]);
    std::vector<int> lens;
    for (int i = 4; i < argc; i++) lens.push_back(std::atoi(argv[i]));
    const int batch = (int)lens.size(), tokens = std::accumulate(lens.begin(), lens.end(), 0);
    const int head_num = 32, kv_heads = 32, head_size = 128, inter = 11008, hidden = head_num * head_size;
    const int max_k = history + *std::max_element(lens.begin(), lens.end()), max_seq = history + max_q;
    try {
        HipAllocator allocator;
        LLaMAAttentionStaticParams params;
        LlamaLayerWeight<half> w(head_num, kv_heads, head_size, inter, WeightType::FP16_W, false);
        w.loadWeights();
        LlamaContextDecoderLayer<half> layer(head_num, kv_heads, head_size, inter, params, 1e-5f, &allocator);
        std::vector<half> rows((size_t)tokens * hidden);
        for (size_t i = 0; i < rows.size(); i++) rows[i] = __float2half((float)((i * 2654435761u >> 16) & 1023) / 512.0f - 1.0f);
        half* residual = upload(rows);
        half* normed = upload(rows);
        half* out = upload(rows);
        const size_t cache_elems = (size_t)batch * kv_heads * max_seq * head_size;
        std::vector<half> past(cache_elems);
        for (size_t i = 0; i < past.size(); i++) past[i] = __float2half((float)((i * 2246822519u >> 16) & 1023) / 512.0f - 1.0f);
        half* k_cache = upload(past);
        half* v_cache = upload(past);
        int* d_lens = upload(lens);
        int* d_hist = upload(std::vector<int>(batch, history));
        std::vector<int> ctx(lens);
        for (int& c : ctx) c += history;
        int* d_ctx = upload(ctx);
        int* d_po = upload(std::vector<int>((size_t)batch * max_q, 0));
        int* d_cum = upload(std::vector<int>(batch + 1, 0));
        TensorWrapper<int> po(Device::GPU, getTensorType<int>(), {batch, max_q}, d_po);
        TensorWrapper<int> cum(Device::GPU, getTensorType<int>(), {batch + 1}, d_cum);
        TensorWrapper<int> il(Device::GPU, getTensorType<int>(), {batch}, d_lens);
        TensorWrapper<int> hl(Device::GPU, getTensorType<int>(), {batch}, d_hist);
        TensorWrapper<int> cl(Device::GPU, getTensorType<int>(), {batch}, d_ctx);
        launchCalPaddingoffset(&po, &cum, &il);
        const DataType dt = getTensorType<half>();
        TensorWrapper<half> in(Device::GPU, dt, {tokens, hidden}, normed);
        TensorWrapper<half> res(Device::GPU, dt, {tokens, hidden}, residual);
        TensorWrapper<half> o(Device::GPU, dt, {tokens, hidden}, out);
        int layer_value = 0;
        TensorWrapper<int> lid(Device::CPU, getTensorType<int>(), {1}, &layer_value);
        TensorWrapper<half> kc(Device::GPU, dt, {1, batch, kv_heads, max_seq, head_size}, k_cache);
        TensorWrapper<half> vc(Device::GPU, dt, {1, batch, kv_heads, max_seq, head_size}, v_cache);
        TensorMap inputs{{"decoder_input", &in}, {"decoder_residual", &res}, {"padding_offset", &po},
                         {"history_length", &hl}, {"input_length", &il}, {"context_length", &cl}, {"layer_id", &lid}};
        TensorMap outputs{{"decoder_output", &o}, {"all_k_cache", &kc}, {"all_v_cache", &vc}};
        LLaMAAttentionDynParams dyn;
        dyn.batch_size = batch, dyn.num_tokens = tokens, dyn.max_q_len = max_q, dyn.max_k_len = max_k, dyn.num_layers = 1;
        auto step = [&] {
            // the layer consumes decoder_input: the previous iteration's output (unit RMS) becomes the next
            // input, one 24 MB device-to-device copy inside the timed region
            CHECK(hipMemcpyAsync(normed, out, rows.size() * sizeof(half), hipMemcpyDeviceToDevice, nullptr));
            layer.forward(inputs, w, w.attn_norm_weight, outputs, dyn);
        };
        for (int i = 0; i < warmup; i++) step();
        CHECK(hipDeviceSynchronize());
        hipEvent_t e0, e1;
        CHECK(hipEventCreate(&e0));
        CHECK(hipEventCreate(&e1));
        CHECK(hipEventRecord(e0, nullptr));
        for (int i = 0; i < iterations; i++) step();
        CHECK(hipEventRecord(e1, nullptr));
        CHECK(hipEventSynchronize(e1));
        float ms = 0.f;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        ms /= (float)iterations;
        std::printf("{\"workload\": \"llama2_7b_context_decoder_layer_f16_cpp\", \"valid_tokens\": %d, \"batch\": %d, "
                    "\"max_q_len\": %d, \"history\": %d, \"ms_per_layer\": %.6f, \"tokens_per_s_per_layer\": %.1f, \"iterations\": %d, "
                    "\"activation_buffer_bytes\": %zu, "
                    "\"attention\": \"%s\", "
                    "\"note\": \"C++ LlamaContextDecoderLayer: launch* kernels + hipBLASLt GEMMs; attention fused on the matrix cores for fp16 heads of 128 or 64 unless ISP_LAYERS_ATTENTION=padded\"}\n",
                    tokens, batch, max_q, history, ms, tokens / (ms * 1e-3), iterations, layer.workspaceBytes(dyn), attention_kind());
    } catch (const std::exception& e) {
        std::printf("exception: %s\n", e.what());
        return 1;
    }
    return 0;
}
