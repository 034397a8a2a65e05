// Call site of the C++ context-decoder layer (LlamaContextDecoderLayer over TensorMap / LlamaLayerWeight /
// BaseAllocator).  The program builds a small ragged batch, runs one layer, and writes every operand and
// result as raw little-endian float32 files into a directory; tests/test_cpp_context_layer.py reads them
// back and checks the results against an independent float64 implementation of the same layer.  A second
// case checks, inside the program, that two turns through the KV cache reproduce one long prefill.
//
//   test_context_layer <f32|f16> <directory> [head_num kv_head_num head_size inter_size]
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <memory>
#include <numeric>
#include <string>

#include "src/kernels/cal_paddingoffset.h"
#include "src/kernels/rmsnorm.h"
#include "src/layers/decoder/context_decoder.h"
#include "src/layers/decoder/context_decoder_layer.h"
#include "src/memory/allocator/hip_allocator.h"
#include "test_util.h"

template <typename T>
static void dump(const std::string& dir, const char* name, const T* device, size_t n) {
    using S = typename Host<T>::Store;
    auto h = to_host(reinterpret_cast<const S*>(device), n);
    std::vector<float> f(n);
    for (size_t i = 0; i < n; i++) f[i] = Host<T>::from(h[i]);
    const std::string path = dir + "/" + name + ".bin";
    FILE* fp = std::fopen(path.c_str(), "wb");
    if (!fp || std::fwrite(f.data(), sizeof(float), n, fp) != n) {
        std::printf("cannot write %s\n", path.c_str());
        std::exit(2);
    }
    std::fclose(fp);
}

template <typename T>
struct Batch {
    int batch, max_q, tokens, max_k;
    int *lens, *hist, *ctx, *padding_offset, *cum;
    Batch(const std::vector<int>& l, const std::vector<int>& h, int max_q_len) : batch((int)l.size()), max_q(max_q_len) {
        tokens = std::accumulate(l.begin(), l.end(), 0);
        std::vector<int> c(batch);
        max_k = 0;
        for (int b = 0; b < batch; b++) {
            c[b] = l[b] + h[b];
            max_k = std::max(max_k, c[b]);
        }
        lens = to_device(l);
        hist = to_device(h);
        ctx = to_device(c);
        padding_offset = to_device(std::vector<int>((size_t)batch * max_q, 0));
        cum = to_device(std::vector<int>(batch + 1, 0));
        TensorWrapper<int> po(Device::GPU, getTensorType<int>(), {batch, max_q}, padding_offset);
        TensorWrapper<int> cs(Device::GPU, getTensorType<int>(), {batch + 1}, cum);
        TensorWrapper<int> il(Device::GPU, getTensorType<int>(), {batch}, lens);
        launchCalPaddingoffset(&po, &cs, &il);
    }
};

// Runs one layer on `rows` (packed [tokens, hidden], storage type); returns through the device buffers.
template <typename T>
static void run_layer(LlamaContextDecoderLayer<T>& layer, LlamaLayerWeight<T>& w, LayerNormWeight<T>& next,
                      Batch<T>& bt, T* residual, T* normed, T* out, T* k_cache, T* v_cache, int layers, int kv_heads,
                      int max_seq, int head_size, int hidden, int layer_index) {
    const DataType dt = getTensorType<T>();
    CHECK(hipMemcpy(normed, residual, (size_t)bt.tokens * hidden * sizeof(T), hipMemcpyDeviceToDevice));
    TensorWrapper<T> in(Device::GPU, dt, {bt.tokens, hidden}, normed);
    launchRMSNorm(&in, w.attn_norm_weight, 1e-5f);
    TensorWrapper<T> res(Device::GPU, dt, {bt.tokens, hidden}, residual);
    TensorWrapper<T> o(Device::GPU, dt, {bt.tokens, hidden}, out);
    TensorWrapper<int> po(Device::GPU, getTensorType<int>(), {bt.batch, bt.max_q}, bt.padding_offset);
    TensorWrapper<int> hl(Device::GPU, getTensorType<int>(), {bt.batch}, bt.hist);
    TensorWrapper<int> il(Device::GPU, getTensorType<int>(), {bt.batch}, bt.lens);
    TensorWrapper<int> cl(Device::GPU, getTensorType<int>(), {bt.batch}, bt.ctx);
    int layer_value = layer_index;
    TensorWrapper<int> lid(Device::CPU, getTensorType<int>(), {1}, &layer_value);
    TensorWrapper<T> kc(Device::GPU, dt, {layers, bt.batch, kv_heads, max_seq, head_size}, k_cache);
    TensorWrapper<T> vc(Device::GPU, dt, {layers, bt.batch, kv_heads, max_seq, head_size}, v_cache);
    TensorMap inputs{{"decoder_input", &in}, {"decoder_residual", &res}, {"padding_offset", &po},
                     {"history_length", &hl}, {"input_length", &il}, {"context_length", &cl}, {"layer_id", &lid}};
    TensorMap outputs{{"decoder_output", &o}, {"all_k_cache", &kc}, {"all_v_cache", &vc}};
    LLaMAAttentionDynParams dyn;
    dyn.batch_size = bt.batch;
    dyn.num_tokens = bt.tokens;
    dyn.max_q_len = bt.max_q;
    dyn.max_k_len = bt.max_k;
    dyn.num_layers = layers;
    layer.forward(inputs, w, next, outputs, dyn);
    CHECK(hipDeviceSynchronize());
}

template <typename T>
static int run(const std::string& dir, int head_num, int kv_heads, int head_size, int inter) {
    using S = typename Host<T>::Store;
    const int hidden = head_num * head_size, layers = 2, max_seq = 32, max_q = 16;
    HipAllocator allocator;
    LLaMAAttentionStaticParams params;
    params.rotary_embedding_dim = head_size;
    LlamaLayerWeight<T> w(head_num, kv_heads, head_size, inter, getWeightType<T>(), /*attn_bias=*/true);
    w.loadWeights();
    std::mt19937 gen(17);
    LayerNormWeight<T> next;
    next.gamma = (T*)to_device(randn<T>(hidden, 0.25f, gen, 1.0f));
    LlamaContextDecoderLayer<T> layer(head_num, kv_heads, head_size, inter, params, 1e-5f, &allocator);

    // ---- case 1: ragged batch, checked by the Python side against float64
    const std::vector<int> lens = {16, 5, 11}, hist = {0, 0, 0};
    Batch<T> bt(lens, hist, max_q);
    auto rows = randn<T>((size_t)bt.tokens * hidden, 1.0f, gen);
    T* residual = (T*)to_device(rows);
    T* normed = (T*)to_device(std::vector<S>(rows.size()));
    T* out = (T*)to_device(std::vector<S>(rows.size()));
    const size_t cache_elems = (size_t)layers * bt.batch * kv_heads * max_seq * head_size;
    T* k_cache = (T*)to_device(std::vector<S>(cache_elems));
    T* v_cache = (T*)to_device(std::vector<S>(cache_elems));
    dump<T>(dir, "residual_in", residual, rows.size());
    run_layer(layer, w, next, bt, residual, normed, out, k_cache, v_cache, layers, kv_heads, max_seq, head_size, hidden, 1);
    const int qkv_out = (head_num + 2 * kv_heads) * head_size;
    dump<T>(dir, "attn_norm", w.attn_norm_weight.gamma, hidden);
    dump<T>(dir, "ffn_norm", w.ffn_norm_weight.gamma, hidden);
    dump<T>(dir, "next_norm", next.gamma, hidden);
    dump<T>(dir, "qkv_weight", w.self_attn_weight.qkv.data, (size_t)qkv_out * hidden);
    dump<T>(dir, "qkv_bias", w.self_attn_weight.qkv.bias, qkv_out);
    dump<T>(dir, "o_weight", w.self_attn_weight.output.data, (size_t)hidden * hidden);
    dump<T>(dir, "o_bias", w.self_attn_weight.output.bias, hidden);
    dump<T>(dir, "gate_up_weight", w.ffn_weight.gateAndup.data, (size_t)2 * inter * hidden);
    dump<T>(dir, "down_weight", w.ffn_weight.down.data, (size_t)hidden * inter);
    dump<T>(dir, "residual_out", residual, rows.size());
    dump<T>(dir, "decoder_output", out, rows.size());
    dump<T>(dir, "k_cache", k_cache, cache_elems);
    dump<T>(dir, "v_cache", v_cache, cache_elems);

    // ---- case 2: 9 tokens, then 7 more with history 9, must equal one 16-token prefill
    auto x = randn<T>((size_t)16 * hidden, 1.0f, gen);
    auto once = [&](const std::vector<int>& l, const std::vector<int>& h, const S* src, size_t n_tokens, T* kc, T* vc,
                    std::vector<S>& res_out, std::vector<S>& next_out) {
        Batch<T> b1(l, h, max_q);
        std::vector<S> part(src, src + n_tokens * hidden);
        T* r = (T*)to_device(part);
        T* nrm = (T*)to_device(std::vector<S>(part.size()));
        T* o = (T*)to_device(std::vector<S>(part.size()));
        run_layer(layer, w, next, b1, r, nrm, o, kc, vc, 1, kv_heads, max_seq, head_size, hidden, 0);
        res_out = to_host((S*)r, part.size());
        next_out = to_host((S*)o, part.size());
    };
    const size_t one_cache = (size_t)kv_heads * max_seq * head_size;
    T* kc_a = (T*)to_device(std::vector<S>(one_cache));
    T* vc_a = (T*)to_device(std::vector<S>(one_cache));
    T* kc_b = (T*)to_device(std::vector<S>(one_cache));
    T* vc_b = (T*)to_device(std::vector<S>(one_cache));
    std::vector<S> r_all, o_all, r1, o1, r2, o2;
    once({16}, {0}, x.data(), 16, kc_a, vc_a, r_all, o_all);
    once({9}, {0}, x.data(), 9, kc_b, vc_b, r1, o1);
    once({7}, {9}, x.data() + (size_t)9 * hidden, 7, kc_b, vc_b, r2, o2);
    r1.insert(r1.end(), r2.begin(), r2.end());
    o1.insert(o1.end(), o2.begin(), o2.end());
    double scale_r = 0, scale_o = 0, err_r = 0, err_o = 0;
    for (size_t i = 0; i < r_all.size(); i++) {
        scale_r = std::max(scale_r, std::fabs((double)Host<T>::from(r_all[i])));
        scale_o = std::max(scale_o, std::fabs((double)Host<T>::from(o_all[i])));
        err_r = std::max(err_r, std::fabs((double)Host<T>::from(r_all[i]) - Host<T>::from(r1[i])));
        err_o = std::max(err_o, std::fabs((double)Host<T>::from(o_all[i]) - Host<T>::from(o1[i])));
    }
    const double tol = std::is_same<T, float>::value ? 2e-4 : 2e-2;
    EXPECT(err_r <= tol * scale_r, "two turns: residual differs by %g (scale %g)", err_r, scale_r);
    EXPECT(err_o <= tol * scale_o, "two turns: output differs by %g (scale %g)", err_o, scale_o);
    auto ka = to_host((S*)kc_a, one_cache), kb = to_host((S*)kc_b, one_cache);
    double err_k = 0;
    for (size_t i = 0; i < ka.size(); i++) err_k = std::max(err_k, std::fabs((double)Host<T>::from(ka[i]) - Host<T>::from(kb[i])));
    EXPECT(err_k <= tol * 8.0, "two turns: cached keys differ by %g", err_k);

    // ---- case 3: the decoder stack equals its layers called one by one
    {
        const int stack_layers = 3;
        std::vector<std::unique_ptr<LlamaLayerWeight<T>>> owned;
        std::vector<LlamaLayerWeight<T>*> ws;
        for (int l = 0; l < stack_layers; l++) {
            owned.emplace_back(new LlamaLayerWeight<T>(head_num, kv_heads, head_size, inter, getWeightType<T>(), l == 1));
            owned.back()->loadWeights();
            // distinct norms per layer, so that a layer picking the wrong "next" norm shows
            auto g1 = randn<T>(hidden, 0.25f, gen, 1.0f), g2 = randn<T>(hidden, 0.25f, gen, 1.0f);
            CHECK(hipMemcpy(owned.back()->attn_norm_weight.gamma, g1.data(), hidden * sizeof(S), hipMemcpyHostToDevice));
            CHECK(hipMemcpy(owned.back()->ffn_norm_weight.gamma, g2.data(), hidden * sizeof(S), hipMemcpyHostToDevice));
            ws.push_back(owned.back().get());
        }
        const std::vector<int> l3 = {7, 16, 3}, h3 = {0, 0, 0};
        Batch<T> b3(l3, h3, max_q);
        auto emb = randn<T>((size_t)b3.tokens * hidden, 1.0f, gen);
        const size_t n = emb.size(), cache3 = (size_t)stack_layers * b3.batch * kv_heads * max_seq * head_size;
        // by hand
        T* r = (T*)to_device(emb);
        T* nrm = (T*)to_device(std::vector<S>(n));
        T* o = (T*)to_device(std::vector<S>(n));
        T* kc1 = (T*)to_device(std::vector<S>(cache3));
        T* vc1 = (T*)to_device(std::vector<S>(cache3));
        {
            const DataType dt = getTensorType<T>();
            CHECK(hipMemcpy(nrm, r, n * sizeof(T), hipMemcpyDeviceToDevice));
            TensorWrapper<T> first(Device::GPU, dt, {b3.tokens, hidden}, nrm);
            launchRMSNorm(&first, ws[0]->attn_norm_weight, 1e-5f);
            T *from = nrm, *to = o;
            for (int l = 0; l < stack_layers; l++) {
                TensorWrapper<T> in(Device::GPU, dt, {b3.tokens, hidden}, from), res(Device::GPU, dt, {b3.tokens, hidden}, r);
                TensorWrapper<T> out_t(Device::GPU, dt, {b3.tokens, hidden}, to);
                TensorWrapper<int> po(Device::GPU, getTensorType<int>(), {b3.batch, b3.max_q}, b3.padding_offset);
                TensorWrapper<int> hl(Device::GPU, getTensorType<int>(), {b3.batch}, b3.hist);
                TensorWrapper<int> il(Device::GPU, getTensorType<int>(), {b3.batch}, b3.lens);
                TensorWrapper<int> cl(Device::GPU, getTensorType<int>(), {b3.batch}, b3.ctx);
                int lv = l;
                TensorWrapper<int> lid(Device::CPU, getTensorType<int>(), {1}, &lv);
                TensorWrapper<T> kc(Device::GPU, dt, {stack_layers, b3.batch, kv_heads, max_seq, head_size}, kc1);
                TensorWrapper<T> vc(Device::GPU, dt, {stack_layers, b3.batch, kv_heads, max_seq, head_size}, vc1);
                TensorMap li{{"decoder_input", &in}, {"decoder_residual", &res}, {"padding_offset", &po}, {"history_length", &hl},
                             {"input_length", &il}, {"context_length", &cl}, {"layer_id", &lid}};
                TensorMap lo{{"decoder_output", &out_t}, {"all_k_cache", &kc}, {"all_v_cache", &vc}};
                LLaMAAttentionDynParams dyn;
                dyn.batch_size = b3.batch, dyn.num_tokens = b3.tokens, dyn.max_q_len = b3.max_q, dyn.max_k_len = b3.max_k;
                dyn.num_layers = stack_layers;
                layer.forward(li, *ws[l], l + 1 < stack_layers ? ws[l + 1]->attn_norm_weight : next, lo, dyn);
                std::swap(from, to);
            }
            CHECK(hipDeviceSynchronize());
            if (from != o) CHECK(hipMemcpy(o, from, n * sizeof(T), hipMemcpyDeviceToDevice));
        }
        // through the stack
        T* e2 = (T*)to_device(emb);
        T* o2 = (T*)to_device(std::vector<S>(n));
        T* kc2 = (T*)to_device(std::vector<S>(cache3));
        T* vc2 = (T*)to_device(std::vector<S>(cache3));
        {
            const DataType dt = getTensorType<T>();
            LlamaContextDecoder<T> decoder(head_num, kv_heads, head_size, inter, stack_layers, params, 1e-5f, &allocator);
            TensorWrapper<T> in(Device::GPU, dt, {b3.tokens, hidden}, e2), out_t(Device::GPU, dt, {b3.tokens, hidden}, o2);
            TensorWrapper<int> hl(Device::GPU, getTensorType<int>(), {b3.batch}, b3.hist);
            TensorWrapper<int> il(Device::GPU, getTensorType<int>(), {b3.batch}, b3.lens);
            TensorWrapper<int> cl(Device::GPU, getTensorType<int>(), {b3.batch}, b3.ctx);
            TensorWrapper<T> kc(Device::GPU, dt, {stack_layers, b3.batch, kv_heads, max_seq, head_size}, kc2);
            TensorWrapper<T> vc(Device::GPU, dt, {stack_layers, b3.batch, kv_heads, max_seq, head_size}, vc2);
            TensorMap di{{"decoder_input", &in}, {"history_length", &hl}, {"input_length", &il}, {"context_length", &cl}};
            TensorMap dout{{"decoder_output", &out_t}, {"all_k_cache", &kc}, {"all_v_cache", &vc}};
            LLaMAAttentionDynParams dyn;
            dyn.batch_size = b3.batch, dyn.num_tokens = b3.tokens, dyn.max_q_len = b3.max_q, dyn.max_k_len = b3.max_k;
            dyn.num_layers = stack_layers;
            decoder.forward(di, ws, next, dout, dyn);
            CHECK(hipDeviceSynchronize());
            auto kept = to_host((S*)e2, n);
            EXPECT(std::memcmp(kept.data(), emb.data(), n * sizeof(S)) == 0, "the stack must leave decoder_input unchanged");
            std::vector<LlamaLayerWeight<T>*> too_few(ws.begin(), ws.begin() + 2);
            EXPECT(throws([&] { decoder.forward(di, too_few, next, dout, dyn); }), "a missing layer's weights must throw");
        }
        // the two engines choose their GEMM algorithms by measurement, each for itself, so the comparison allows
        // for a different summation order inside the GEMMs
        auto a = to_host((S*)o, n), b = to_host((S*)o2, n);
        auto worst = [](const std::vector<S>& u, const std::vector<S>& w, double& scale) {
            double err = 0;
            scale = 0;
            for (size_t i = 0; i < u.size(); i++) {
                scale = std::max(scale, std::fabs((double)Host<T>::from(u[i])));
                err = std::max(err, std::fabs((double)Host<T>::from(u[i]) - Host<T>::from(w[i])));
            }
            return err;
        };
        double sc = 0;
        const double tol3 = std::is_same<T, float>::value ? 3e-4 : 3e-2;
        const double eo = worst(a, b, sc);
        EXPECT(eo <= tol3 * sc, "decoder stack: output differs from the layers called by hand by %g (scale %g)", eo, sc);
        auto ka3 = to_host((S*)kc1, cache3), kb3 = to_host((S*)kc2, cache3), va3 = to_host((S*)vc1, cache3), vb3 = to_host((S*)vc2, cache3);
        const double ek = worst(ka3, kb3, sc);
        EXPECT(ek <= tol3 * sc, "decoder stack: cached keys differ by %g (scale %g)", ek, sc);
        const double ev = worst(va3, vb3, sc);
        EXPECT(ev <= tol3 * sc, "decoder stack: cached values differ by %g (scale %g)", ev, sc);
        double peak = 0;
        for (size_t i = 0; i < n; i++) peak = std::max(peak, std::fabs((double)Host<T>::from(b[i])));
        EXPECT(peak > 0.1 && peak < 100.0, "decoder stack: implausible output scale %g", peak);
    }

    // ---- case 4: the attention softmax by itself against float64, at every row width its kernels split on
    {
        struct Shape {
            int batch, heads, max_q, max_k;
        };
        // 16: a few vectors; 100: a whole number of fp32 vectors but not of fp16 ones (the workgroup-per-row kernel);
        // 512 / 1024 / 2048: one, two and four vectors per lane; 1032 and 2056: the last lanes idle; 5 and 7 queries:
        // a last workgroup with idle wavefronts
        const Shape shapes[] = {{3, 2, 5, 16}, {2, 3, 7, 100}, {2, 2, 16, 512}, {2, 1, 9, 1024}, {2, 1, 6, 1032},
                                {1, 2, 5, 2048}, {1, 1, 4, 2056}, {1, 1, 3, 4096}};
        for (const Shape& sh : shapes) {
            std::vector<int> hl(sh.batch), il(sh.batch), cl(sh.batch);
            for (int b = 0; b < sh.batch; b++) {
                il[b] = b == 0 ? sh.max_q : 1 + (int)(gen() % (unsigned)sh.max_q);              // a ragged batch
                hl[b] = b == 0 ? 0 : (int)(gen() % (unsigned)std::max(1, sh.max_k - il[b]));   // some with history
                cl[b] = b == 1 ? std::max(1, hl[b] + il[b] - 1) : hl[b] + il[b];                // one context cut short
                cl[b] = std::min(cl[b], sh.max_k);
            }
            const size_t n = (size_t)sh.batch * sh.heads * sh.max_q * sh.max_k;
            auto in = randn<T>(n, 8.0f, gen);   // scaled by 1/sqrt(128): exponents spread over +-3
            T* d = (T*)to_device(in);
            int* d_hl = (int*)to_device(hl);
            int* d_il = (int*)to_device(il);
            int* d_cl = (int*)to_device(cl);
            const float scale = 0.08838834764831845f;
            isp_layers::launch_masked_scaled_softmax(d, d_hl, d_il, d_cl, sh.batch, sh.heads, sh.max_q, sh.max_k, scale);
            CHECK(hipDeviceSynchronize());
            auto out = to_host((S*)d, n);
            double worst = 0, worst_sum = 0;
            long long leaked = 0;
            for (int b = 0; b < sh.batch; b++)
                for (int h = 0; h < sh.heads; h++)
                    for (int q = 0; q < sh.max_q; q++) {
                        const size_t base = (((size_t)b * sh.heads + h) * sh.max_q + q) * sh.max_k;
                        int visible = 0;
                        if (q < il[b]) visible = std::min(std::min(hl[b] + q + 1, cl[b]), sh.max_k);
                        double m = -1e300, sum = 0, got_sum = 0;
                        for (int k = 0; k < visible; k++) m = std::max(m, (double)scale * Host<T>::from(in[base + k]));
                        for (int k = 0; k < visible; k++) sum += std::exp((double)scale * Host<T>::from(in[base + k]) - m);
                        for (int k = 0; k < sh.max_k; k++) {
                            const double got = Host<T>::from(out[base + k]);
                            if (k >= visible) {
                                leaked += got != 0.0;
                                continue;
                            }
                            const double want = std::exp((double)scale * Host<T>::from(in[base + k]) - m) / sum;
                            worst = std::max(worst, std::fabs(got - want) / (std::is_same<T, float>::value ? want : std::max(want, 1.0 / 1024)));
                            got_sum += got;
                        }
                        if (visible > 0) worst_sum = std::max(worst_sum, std::fabs(got_sum - 1.0));
                    }
            // fp32: the hardware exponential's 2^-22 and the rounding of the scaled difference; fp16: one rounding of the result
            const double tol = std::is_same<T, float>::value ? 4e-6 : 6e-4;
            EXPECT(leaked == 0, "softmax %dx%dx%dx%d: %lld masked probabilities are not exactly zero", sh.batch, sh.heads,
                   sh.max_q, sh.max_k, leaked);
            EXPECT(worst <= tol, "softmax %dx%dx%dx%d: relative error %g", sh.batch, sh.heads, sh.max_q, sh.max_k, worst);
            EXPECT(worst_sum <= (std::is_same<T, float>::value ? 1e-5 : 4e-3), "softmax %dx%dx%dx%d: a row sums to 1 %+g",
                   sh.batch, sh.heads, sh.max_q, sh.max_k, worst_sum);
            CHECK(hipFree(d));
            CHECK(hipFree(d_hl));
            CHECK(hipFree(d_il));
            CHECK(hipFree(d_cl));
        }
    }

    // ---- case 5: weights written as the reference's per-tensor fp32 files load back to the same bits
    {
        const std::string prefix = dir + "/model.layers.0";
        const int qkv_n = (head_num + 2 * kv_heads) * head_size;
        auto write = [&](const char* suffix, const T* device, size_t n) { dump<T>(dir, (std::string("model.layers.0") + suffix).c_str(), device, n); };
        // dump() appends ".bin", the names are the reference's (src/weights/llama/layer_weights.cc:47-57)
        write(".input_layernorm.weight", w.attn_norm_weight.gamma, hidden);
        write(".post_attention_layernorm.weight", w.ffn_norm_weight.gamma, hidden);
        write(".self_attn.qkv.weight", w.self_attn_weight.qkv.data, (size_t)qkv_n * hidden);
        write(".self_attn.o_proj.weight", w.self_attn_weight.output.data, (size_t)hidden * hidden);
        write(".mlp.gate_up_proj.weight", w.ffn_weight.gateAndup.data, (size_t)2 * inter * hidden);
        write(".mlp.down_proj.weight", w.ffn_weight.down.data, (size_t)hidden * inter);
        write(".attention.wqkv.bias", w.self_attn_weight.qkv.bias, qkv_n);
        write(".attention.wo.bias", w.self_attn_weight.output.bias, hidden);
        auto same = [&](const T* a, const T* b, size_t n) {
            auto x = to_host((const S*)a, n), y = to_host((const S*)b, n);
            return std::memcmp(x.data(), y.data(), n * sizeof(S)) == 0;
        };
        LlamaLayerWeight<T> loaded(head_num, kv_heads, head_size, inter, getWeightType<T>(), /*attn_bias=*/true);
        loaded.loadWeights(prefix, getWeightType<T>());
        EXPECT(same(loaded.attn_norm_weight.gamma, w.attn_norm_weight.gamma, hidden) &&
                   same(loaded.ffn_norm_weight.gamma, w.ffn_norm_weight.gamma, hidden) &&
                   same(loaded.self_attn_weight.qkv.data, w.self_attn_weight.qkv.data, (size_t)qkv_n * hidden) &&
                   same(loaded.self_attn_weight.output.data, w.self_attn_weight.output.data, (size_t)hidden * hidden) &&
                   same(loaded.ffn_weight.gateAndup.data, w.ffn_weight.gateAndup.data, (size_t)2 * inter * hidden) &&
                   same(loaded.ffn_weight.down.data, w.ffn_weight.down.data, (size_t)hidden * inter) &&
                   same(loaded.self_attn_weight.qkv.bias, w.self_attn_weight.qkv.bias, qkv_n) &&
                   same(loaded.self_attn_weight.output.bias, w.self_attn_weight.output.bias, hidden),
               "weights loaded from files differ from the ones written");
        LlamaLayerWeight<T> no_bias(head_num, kv_heads, head_size, inter, getWeightType<T>(), /*attn_bias=*/false);
        no_bias.loadWeights(prefix, getWeightType<T>());
        EXPECT(no_bias.self_attn_weight.qkv.bias == nullptr && no_bias.self_attn_weight.output.bias == nullptr &&
                   no_bias.ffn_weight.down.bias == nullptr,
               "without attn_bias the loader must leave every bias null");
        EXPECT(same(no_bias.ffn_weight.down.data, w.ffn_weight.down.data, (size_t)hidden * inter), "down weight without bias");
        EXPECT(throws([&] { loaded.loadWeights(dir + "/no.such.layer", getWeightType<T>()); }), "a missing weight file must throw");
    }

    // ---- case 6: after a call at the largest extents the layer takes nothing more from the allocator
    {
        struct Counting : HipAllocator {
            int mallocs = 0;
            void* UnifyMalloc(void* ptr, size_t size, bool is_host = false) override {
                mallocs++;
                return HipAllocator::UnifyMalloc(ptr, size, is_host);
            }
        } counting;
        {
            LlamaContextDecoderLayer<T> fresh(head_num, kv_heads, head_size, inter, params, 1e-5f, &counting);
            const size_t one = (size_t)3 * kv_heads * max_seq * head_size;
            T* kc6 = (T*)to_device(std::vector<S>(one));
            T* vc6 = (T*)to_device(std::vector<S>(one));
            auto call = [&](const std::vector<int>& l, const std::vector<int>& h, std::vector<S>& next_out) {
                Batch<T> b6(l, h, *std::max_element(l.begin(), l.end()));
                std::vector<S> part(rows.begin(), rows.begin() + (size_t)b6.tokens * hidden);
                T* r = (T*)to_device(part);
                T* nrm = (T*)to_device(std::vector<S>(part.size()));
                T* o = (T*)to_device(std::vector<S>(part.size()));
                run_layer(fresh, w, next, b6, r, nrm, o, kc6, vc6, 1, kv_heads, max_seq, head_size, hidden, 0);
                next_out = to_host((S*)o, part.size());
                CHECK(hipFree(r));
                CHECK(hipFree(nrm));
                CHECK(hipFree(o));
            };
            std::vector<S> big, small_after, small_alone;
            call({16, 5, 11}, {0, 0, 0}, big);
            const int after_first = counting.mallocs;
            EXPECT(after_first > 0, "the first call must allocate the layer's buffers");
            call({4, 9}, {0, 0}, small_after);          // fewer sequences, shorter, other padded extents
            call({16, 5, 11}, {0, 0, 0}, big);
            call({1, 1, 1}, {7, 2, 9}, small_after);    // a decode-shaped call: one token each, longer contexts
            call({4, 9}, {0, 0}, small_after);
            EXPECT(counting.mallocs == after_first, "later, smaller calls allocated %d more buffers", counting.mallocs - after_first);
            // ... and a buffer that held a larger batch gives the results of a layer that never saw one
            LlamaContextDecoderLayer<T> clean(head_num, kv_heads, head_size, inter, params, 1e-5f, &allocator);
            T* kc7 = (T*)to_device(std::vector<S>(one));
            T* vc7 = (T*)to_device(std::vector<S>(one));
            {
                Batch<T> b7({4, 9}, {0, 0}, 9);
                std::vector<S> part(rows.begin(), rows.begin() + (size_t)b7.tokens * hidden);
                T* r = (T*)to_device(part);
                T* nrm = (T*)to_device(std::vector<S>(part.size()));
                T* o = (T*)to_device(std::vector<S>(part.size()));
                run_layer(clean, w, next, b7, r, nrm, o, kc7, vc7, 1, kv_heads, max_seq, head_size, hidden, 0);
                small_alone = to_host((S*)o, part.size());
            }
            double err = 0, scale = 0;
            for (size_t i = 0; i < small_alone.size(); i++) {
                scale = std::max(scale, std::fabs((double)Host<T>::from(small_alone[i])));
                err = std::max(err, std::fabs((double)Host<T>::from(small_alone[i]) - Host<T>::from(small_after[i])));
            }
            // each layer object measures its GEMM algorithms for itself: allow for another summation order
            EXPECT(err <= (std::is_same<T, float>::value ? 3e-4 : 3e-2) * scale, "reused buffers change the result by %g (scale %g)", err, scale);
        }
    }

    // ---- the layer rejects tensors that do not fit
    {
        Batch<T> b2(lens, hist, max_q);
        T* r = (T*)to_device(rows);
        TensorWrapper<T> bad(Device::GPU, getTensorType<T>(), {bt.tokens, hidden + 1}, r);
        TensorWrapper<T> good(Device::GPU, getTensorType<T>(), {bt.tokens, hidden}, r);
        TensorWrapper<int> po(Device::GPU, getTensorType<int>(), {bt.batch, bt.max_q}, b2.padding_offset);
        TensorWrapper<int> hl(Device::GPU, getTensorType<int>(), {bt.batch}, b2.hist);
        int lv = 0;
        TensorWrapper<int> lid(Device::CPU, getTensorType<int>(), {1}, &lv);
        TensorWrapper<T> kc(Device::GPU, getTensorType<T>(), {layers, bt.batch, kv_heads, max_seq, head_size}, k_cache);
        TensorMap inputs{{"decoder_input", &bad}, {"decoder_residual", &good}, {"padding_offset", &po}, {"history_length", &hl},
                         {"input_length", &hl}, {"context_length", &hl}, {"layer_id", &lid}};
        TensorMap outputs{{"decoder_output", &good}, {"all_k_cache", &kc}, {"all_v_cache", &kc}};
        LLaMAAttentionDynParams dyn;
        dyn.batch_size = bt.batch, dyn.num_tokens = bt.tokens, dyn.max_q_len = max_q, dyn.max_k_len = 16;
        EXPECT(throws([&] { layer.forward(inputs, w, next, outputs, dyn); }), "a mis-shaped decoder_input must throw");
        TensorMap missing{{"decoder_input", &good}};
        EXPECT(throws([&] { layer.forward(missing, w, next, outputs, dyn); }), "a missing input must throw");
    }
    std::printf("context layer %s: %d tokens, hidden %d, %d/%d heads x %d, inter %d: %s\n",
                std::is_same<T, float>::value ? "f32" : "f16", bt.tokens, hidden, head_num, kv_heads, head_size, inter,
                g_failures ? "FAILED" : "passed");
    return g_failures;
}

int main(int argc, char** argv) {
    if (argc < 3) {
        std::printf("usage: test_context_layer <f32|f16> <directory> [head_num kv_head_num head_size inter_size]\n");
        return 2;
    }
    const std::string type = argv[1], dir = argv[2];
    const int head_num = argc > 6 ? std::atoi(argv[3]) : 2, kv = argc > 6 ? std::atoi(argv[4]) : 2;
    const int hs = argc > 6 ? std::atoi(argv[5]) : 128, inter = argc > 6 ? std::atoi(argv[6]) : 512;
    try {
        return type == "f16" ? run<half>(dir, head_num, kv, hs, inter) : run<float>(dir, head_num, kv, hs, inter);
    } catch (const std::exception& e) {
        std::printf("exception: %s\n", e.what());
        return 1;
    }
}
