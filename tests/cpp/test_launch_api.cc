// Reference-style call sites for the C++ launch* entry points: every case builds TensorWrapper /
// weight structs exactly as the reference's tests/unittests/*.cu programs do, calls the launcher,
// copies the result back and checks it -- against the CPU oracle on seeded random inputs and against
// the known answers those reference programs state.  Unlike the reference's programs, a mismatch
// fails the process.
//
//   test_launch_api <case>      case = embedding | padding | norm | rmsnorm | qkv | act | bias_modes | errors | all
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <map>
#include <random>
#include <string>
#include <vector>

#include "inferspore_amd_shims.h"
#include "isp_oracle.h"
#include "src/kernels/act_kernel.h"
#include "src/kernels/cal_paddingoffset.h"
#include "src/kernels/fused_addresidual_norm.h"
#include "src/kernels/input_embedding.h"
#include "src/kernels/qkv_bias_and_RoPE.h"
#include "src/kernels/rmsnorm.h"
#include "src/weights/llama/attention_weights.h"

#include "test_util.h"

// --------------------------------------------------------------------------- embedding
template <typename T>
void case_embedding() {
    using S = typename Host<T>::Store;
    const int tokens = 64, hidden = 4096, vocab = 32000;  // reference test sizes
    std::mt19937 gen(1);
    std::uniform_int_distribution<int> pick(0, vocab - 1);
    std::vector<int> ids(tokens);
    for (auto& i : ids) i = pick(gen);
    std::vector<S> table((size_t)vocab * hidden);
    for (size_t i = 0; i < table.size(); i++) table[i] = Host<T>::to((float)(i / hidden));  // table[r, :] = r
    int* d_ids = to_device(ids);
    S* d_table = to_device(table);
    S* d_out = to_device(std::vector<S>((size_t)tokens * hidden));
    TensorWrapper<int>* input_ids = new TensorWrapper<int>(Device::GPU, getTensorType<int>(), {tokens}, d_ids);
    TensorWrapper<T>* output = new TensorWrapper<T>(Device::GPU, getTensorType<T>(), {tokens, hidden}, (T*)d_out);
    EmbeddingWeight<T> emb_table;
    emb_table.data = (T*)d_table;
    launchInputEmbedding(input_ids, output, &emb_table);
    auto out = to_host(d_out, (size_t)tokens * hidden);
    std::vector<S> ref(out.size());
    isp_oracle_embedding(ids.data(), ref.data(), table.data(), tokens, hidden, sizeof(S));
    EXPECT(std::memcmp(out.data(), ref.data(), out.size() * sizeof(S)) == 0, "embedding differs from the oracle");
    for (int t = 0; t < tokens; t++)  // the reference's printed check: out[t, 0] == ids[t]
        EXPECT(Host<T>::from(out[(size_t)t * hidden]) == Host<T>::from(Host<T>::to((float)ids[t])), "row %d", t);
    hipFree(d_ids); hipFree(d_table); hipFree(d_out);
}

// --------------------------------------------------------------------------- padding offset
void case_padding() {
    const int batch_size = 3, max_q_len = 5;  // reference test: lens 3,3,3
    std::vector<int> lens(batch_size, 3);
    int* d_lens = to_device(lens);
    int* d_po = to_device(std::vector<int>(batch_size * max_q_len, -1));
    int* d_cum = to_device(std::vector<int>(batch_size + 1, -1));
    TensorWrapper<int>* padding_offset = new TensorWrapper<int>(Device::GPU, getTensorType<int>(), {batch_size, max_q_len}, d_po);
    TensorWrapper<int>* cum_seqlens = new TensorWrapper<int>(Device::GPU, getTensorType<int>(), {batch_size + 1}, d_cum);
    TensorWrapper<int>* input_lengths = new TensorWrapper<int>(Device::GPU, getTensorType<int>(), {batch_size}, d_lens);
    launchCalPaddingoffset(padding_offset, cum_seqlens, input_lengths);
    auto po = to_host(d_po, batch_size * max_q_len);
    auto cum = to_host(d_cum, batch_size + 1);
    const int expect_po[9] = {0, 0, 0, 2, 2, 2, 4, 4, 4};
    for (int i = 0; i < 9; i++) EXPECT(po[i] == expect_po[i], "padding_offset[%d] = %d", i, po[i]);
    for (int i = 9; i < 15; i++) EXPECT(po[i] == -1, "padding_offset[%d] was written", i);
    const int expect_cum[4] = {0, 3, 6, 9};
    for (int i = 0; i < 4; i++) EXPECT(cum[i] == expect_cum[i], "cum_seqlens[%d] = %d", i, cum[i]);
}

// --------------------------------------------------------------------------- fused norm
template <typename T>
void case_norm() {
    using S = typename Host<T>::Store;
    {  // the reference's own case: out = 1, residual = 0, gamma = 1, eps = 0.5, [2, 32]
        const int num_tokens = 2, hidden_units = 32;
        S* d_out = to_device(std::vector<S>(num_tokens * hidden_units, Host<T>::to(1.f)));
        S* d_res = to_device(std::vector<S>(num_tokens * hidden_units, Host<T>::to(0.f)));
        S* d_scale = to_device(std::vector<S>(hidden_units, Host<T>::to(1.f)));
        TensorWrapper<T>* decoder_out_tensor = new TensorWrapper<T>(Device::GPU, getTensorType<T>(), {num_tokens, hidden_units}, (T*)d_out);
        TensorWrapper<T>* residual_tensor = new TensorWrapper<T>(Device::GPU, getTensorType<T>(), {num_tokens, hidden_units}, (T*)d_res);
        BaseWeight<T> norm;  // bias left unset, as in the reference test
        launchFusedAddBiasResidualRMSNorm(residual_tensor, decoder_out_tensor, norm, (T*)d_scale, 0.5f);
        auto out = to_host(d_out, num_tokens * hidden_units);
        const float expect = Host<T>::from(Host<T>::to(0.816496580927726f));
        for (size_t i = 0; i < out.size(); i++)
            EXPECT(std::fabs(Host<T>::from(out[i]) - expect) <= 1e-6f, "known answer [%zu] = %g", i, Host<T>::from(out[i]));
    }
    const int tokens = 129, hidden = 4096;
    std::mt19937 gen(2);
    auto out = randn<T>((size_t)tokens * hidden, 1.f, gen);
    auto res = randn<T>((size_t)tokens * hidden, 1.f, gen);
    auto bias = randn<T>(hidden, 0.02f, gen);
    auto gamma = randn<T>(hidden, 0.25f, gen, 1.0f);
    S *d_out = to_device(out), *d_res = to_device(res), *d_bias = to_device(bias), *d_gamma = to_device(gamma);
    TensorWrapper<T> out_t(Device::GPU, getTensorType<T>(), {tokens, hidden}, (T*)d_out);
    TensorWrapper<T> res_t(Device::GPU, getTensorType<T>(), {tokens, hidden}, (T*)d_res);
    BaseWeight<T> norm;
    norm.bias = (T*)d_bias;
    launchFusedAddBiasResidualRMSNorm(&res_t, &out_t, norm, (T*)d_gamma, 1e-5f);
    if (std::is_same<T, float>::value)
        isp_oracle_fused_norm_f32((float*)res.data(), (float*)out.data(), (const float*)bias.data(), (const float*)gamma.data(), 1e-5f, tokens, hidden, 0);
    else
        isp_oracle_fused_norm_f16((uint16_t*)res.data(), (uint16_t*)out.data(), (const uint16_t*)bias.data(), (const uint16_t*)gamma.data(), 1e-5f, tokens, hidden, 0);
    compare<T>(to_host(d_out, out.size()), out, "normalised output");
    auto got_res = to_host(d_res, res.size());
    EXPECT(std::memcmp(got_res.data(), res.data(), res.size() * sizeof(S)) == 0, "residual differs from the oracle");
}

template <typename T>
void case_rmsnorm() {
    using S = typename Host<T>::Store;
    const int tokens = 64, hidden = 4096;
    std::mt19937 gen(3);
    auto x = randn<T>((size_t)tokens * hidden, 1.f, gen);
    auto gamma = randn<T>(hidden, 0.25f, gen, 1.0f);
    S *d_x = to_device(x), *d_gamma = to_device(gamma);
    TensorWrapper<T> x_t(Device::GPU, getTensorType<T>(), {tokens, hidden}, (T*)d_x);
    LayerNormWeight<T> w;
    w.gamma = (T*)d_gamma;
    launchRMSNorm(&x_t, w, 1e-5f);
    // the in-tree route of the reference: null residual data and null bias through the fused launcher
    S* d_x2 = to_device(x);
    TensorWrapper<T> x2_t(Device::GPU, getTensorType<T>(), {tokens, hidden}, (T*)d_x2);
    TensorWrapper<T> no_residual(Device::GPU, getTensorType<T>(), {tokens, hidden}, nullptr);
    BaseWeight<T> norm;
    launchFusedAddBiasResidualRMSNorm(&no_residual, &x2_t, norm, (T*)d_gamma, 1e-5f);
    if (std::is_same<T, float>::value)
        isp_oracle_fused_norm_f32(nullptr, (float*)x.data(), nullptr, (const float*)gamma.data(), 1e-5f, tokens, hidden, 0);
    else
        isp_oracle_fused_norm_f16(nullptr, (uint16_t*)x.data(), nullptr, (const uint16_t*)gamma.data(), 1e-5f, tokens, hidden, 0);
    auto a = to_host(d_x, x.size()), b = to_host(d_x2, x.size());
    compare<T>(a, x, "rmsnorm");
    EXPECT(std::memcmp(a.data(), b.data(), a.size() * sizeof(S)) == 0, "launchRMSNorm and the fused route differ");
}

// --------------------------------------------------------------------------- qkv + rope
template <typename T>
void case_qkv() {
    using S = typename Host<T>::Store;
    {  // the reference's own case (fp32 there): QKV = 32, no padding, history 0, seq 32
        const int batch_size = 1, seq_len = 32, token_num = 32, head_num = 32, kv_head_num = 32, head_size = 128;
        const size_t qn = (size_t)batch_size * seq_len * head_num * head_size;
        S* dq = to_device(std::vector<S>(qn));
        S* dk = to_device(std::vector<S>(qn));
        S* dv = to_device(std::vector<S>(qn));
        S* dQKV = to_device(std::vector<S>((size_t)token_num * 96 * head_size, Host<T>::to(32.f)));
        int* dpad = to_device(std::vector<int>(batch_size * seq_len, 0));
        int* dhist = to_device(std::vector<int>(batch_size, 0));
        int* dlen = to_device(std::vector<int>(batch_size, 7));
        TensorWrapper<T>* q_buf = new TensorWrapper<T>(Device::GPU, getTensorType<T>(), {batch_size, head_num, seq_len, head_size}, (T*)dq);
        TensorWrapper<T>* k_buf = new TensorWrapper<T>(Device::GPU, getTensorType<T>(), {batch_size, kv_head_num, seq_len, head_size}, (T*)dk);
        TensorWrapper<T>* v_buf = new TensorWrapper<T>(Device::GPU, getTensorType<T>(), {batch_size, kv_head_num, seq_len, head_size}, (T*)dv);
        TensorWrapper<T>* QKV_buf = new TensorWrapper<T>(Device::GPU, getTensorType<T>(), {token_num, head_num + 2 * kv_head_num, head_size}, (T*)dQKV);
        LLaMAattentionWeights<T> attn_weights;  // qkv.bias stays null: the reference's fp32 kernel ignores it
        TensorWrapper<int>* input_length_buf = new TensorWrapper<int>(Device::GPU, getTensorType<int>(), {batch_size}, dlen);
        TensorWrapper<int>* history_length_buf = new TensorWrapper<int>(Device::GPU, getTensorType<int>(), {batch_size}, dhist);
        TensorWrapper<int>* padding_offset_buf = new TensorWrapper<int>(Device::GPU, getTensorType<int>(), {batch_size, seq_len}, dpad);
        LLaMAAttentionStaticParams params;
        params.rotary_embedding_dim = 128;
        params.rotary_embedding_base = 10000;
        params.max_position_embeddings = 2048;
        params.use_dynamic_ntk = false;
        launchAddFusedQKVBiasTransposeAndRoPE(q_buf, k_buf, v_buf, QKV_buf, attn_weights.qkv, padding_offset_buf,
                                              history_length_buf, input_length_buf, params);
        auto q = to_host(dq, qn), k = to_host(dk, qn), v = to_host(dv, qn);
        const double tol = std::is_same<T, float>::value ? 32 * 1.5 * 1e-5 : 2 * f16_ulp(45.0);
        for (int h = 0; h < head_num; h += 7)
            for (int s = 0; s < seq_len; s++)
                for (int d = 0; d < 64; d++) {
                    const double a = s / std::pow(10000.0, d / 64.0);
                    const size_t i = ((size_t)h * seq_len + s) * head_size + d;
                    EXPECT(std::fabs(Host<T>::from(q[i]) - 32 * (std::cos(a) - std::sin(a))) <= tol, "q[%d,%d,%d]", h, s, d);
                    EXPECT(std::fabs(Host<T>::from(k[i + 64]) - 32 * (std::cos(a) + std::sin(a))) <= tol, "k[%d,%d,%d]", h, s, d + 64);
                    EXPECT(Host<T>::from(v[i]) == 32.f, "v[%d,%d,%d]", h, s, d);
                }
    }
    // ragged batch with bias and history against the oracle
    const int batch = 3, seq = 24, hn = 32, kvn = 32, hs = 128;
    const std::vector<int> lens = {24, 7, 15}, hist = {0, 100, 3};
    int tokens = 0;
    for (int l : lens) tokens += l;
    std::mt19937 gen(4);
    auto qkv = randn<T>((size_t)tokens * (hn + 2 * kvn) * hs, 1.f, gen);
    auto bias = randn<T>((size_t)(hn + 2 * kvn) * hs, 0.02f, gen);
    int* d_lens = to_device(lens);
    int* d_hist = to_device(hist);
    int* d_po = to_device(std::vector<int>(batch * seq, 0));
    int* d_cum = to_device(std::vector<int>(batch + 1, 0));
    TensorWrapper<int> po_t(Device::GPU, getTensorType<int>(), {batch, seq}, d_po);
    TensorWrapper<int> cum_t(Device::GPU, getTensorType<int>(), {batch + 1}, d_cum);
    TensorWrapper<int> lens_t(Device::GPU, getTensorType<int>(), {batch}, d_lens);
    TensorWrapper<int> hist_t(Device::GPU, getTensorType<int>(), {batch}, d_hist);
    launchCalPaddingoffset(&po_t, &cum_t, &lens_t);
    const size_t qn = (size_t)batch * hn * seq * hs;
    const S sentinel = Host<T>::to(-77.f);
    S *dq = to_device(std::vector<S>(qn, sentinel)), *dk = to_device(std::vector<S>(qn, sentinel)), *dv = to_device(std::vector<S>(qn, sentinel));
    S *d_qkv = to_device(qkv), *d_bias = to_device(bias);
    TensorWrapper<T> q_t(Device::GPU, getTensorType<T>(), {batch, hn, seq, hs}, (T*)dq);
    TensorWrapper<T> k_t(Device::GPU, getTensorType<T>(), {batch, kvn, seq, hs}, (T*)dk);
    TensorWrapper<T> v_t(Device::GPU, getTensorType<T>(), {batch, kvn, seq, hs}, (T*)dv);
    TensorWrapper<T> qkv_t(Device::GPU, getTensorType<T>(), {tokens, hn + 2 * kvn, hs}, (T*)d_qkv);
    BaseWeight<T> w;
    w.bias = (T*)d_bias;
    LLaMAAttentionStaticParams params;
    launchAddFusedQKVBiasTransposeAndRoPE(&q_t, &k_t, &v_t, &qkv_t, w, &po_t, &hist_t, &lens_t, params);
    std::vector<int> po(batch * seq, 0), cum(batch + 1, 0);
    isp_oracle_cal_padding_offset(po.data(), cum.data(), lens.data(), batch, seq);
    std::vector<S> eq(qn, sentinel), ek(qn, sentinel), ev(qn, sentinel);
    if (std::is_same<T, float>::value)
        isp_oracle_qkv_rope_f32((float*)eq.data(), (float*)ek.data(), (float*)ev.data(), (const float*)qkv.data(), (const float*)bias.data(),
                                po.data(), hist.data(), lens.data(), batch, seq, tokens, hn, kvn, hs, 128, 10000.f);
    else
        isp_oracle_qkv_rope_f16((uint16_t*)eq.data(), (uint16_t*)ek.data(), (uint16_t*)ev.data(), (const uint16_t*)qkv.data(),
                                (const uint16_t*)bias.data(), po.data(), hist.data(), lens.data(), batch, seq, tokens, hn, kvn, hs, 128, 10000.f);
    auto mag = [](size_t) { return 6.0; };  // |x| <= ~4.5 per component: bounds the radius of every rotated pair
    compare<T>(to_host(dq, qn), eq, "q", mag);
    compare<T>(to_host(dk, qn), ek, "k", mag);
    auto gv = to_host(dv, qn);
    EXPECT(std::memcmp(gv.data(), ev.data(), qn * sizeof(S)) == 0, "v differs from the oracle");
}

// --------------------------------------------------------------------------- the two bias modes
// Non-null biases through the launchers, once as the operators' names say (the default) and once as
// the reference's kernels literally behave (isp_shims::setReferenceLiteralBias): each mode against the
// oracle run in the same mode, and the two modes must differ exactly where the bias enters.
template <typename T>
void case_bias_modes() {
    using S = typename Host<T>::Store;
    const bool before = isp_shims::referenceLiteralBias();
    for (int literal = 0; literal < 2; literal++) {
        isp_shims::setReferenceLiteralBias(literal != 0);
        EXPECT(isp_shims::referenceLiteralBias() == (literal != 0), "setting must read back");
        {   // fused norm: the normalised output includes the bias in both modes, the stored residual only by default
            const int tokens = 33, hidden = 1024;
            std::mt19937 gen(21);
            auto out = randn<T>((size_t)tokens * hidden, 1.f, gen);
            auto res = randn<T>((size_t)tokens * hidden, 1.f, gen);
            auto bias = randn<T>(hidden, 0.5f, gen);
            auto gamma = randn<T>(hidden, 0.25f, gen, 1.0f);
            S *d_out = to_device(out), *d_res = to_device(res), *d_bias = to_device(bias), *d_gamma = to_device(gamma);
            TensorWrapper<T> out_t(Device::GPU, getTensorType<T>(), {tokens, hidden}, (T*)d_out);
            TensorWrapper<T> res_t(Device::GPU, getTensorType<T>(), {tokens, hidden}, (T*)d_res);
            BaseWeight<T> norm;
            norm.bias = (T*)d_bias;
            launchFusedAddBiasResidualRMSNorm(&res_t, &out_t, norm, (T*)d_gamma, 1e-5f);
            auto res_other = res, out_other = out;
            const unsigned flags = literal ? ISP_ORACLE_NORM_RESIDUAL_EXCLUDES_BIAS : 0u;
            if (std::is_same<T, float>::value) {
                isp_oracle_fused_norm_f32((float*)res.data(), (float*)out.data(), (const float*)bias.data(), (const float*)gamma.data(), 1e-5f, tokens, hidden, flags);
                isp_oracle_fused_norm_f32((float*)res_other.data(), (float*)out_other.data(), (const float*)bias.data(), (const float*)gamma.data(), 1e-5f, tokens, hidden, flags ^ 1u);
            } else {
                isp_oracle_fused_norm_f16((uint16_t*)res.data(), (uint16_t*)out.data(), (const uint16_t*)bias.data(), (const uint16_t*)gamma.data(), 1e-5f, tokens, hidden, flags);
                isp_oracle_fused_norm_f16((uint16_t*)res_other.data(), (uint16_t*)out_other.data(), (const uint16_t*)bias.data(), (const uint16_t*)gamma.data(), 1e-5f, tokens, hidden, flags ^ 1u);
            }
            compare<T>(to_host(d_out, out.size()), out, literal ? "literal mode: normalised output" : "default mode: normalised output");
            auto got_res = to_host(d_res, res.size());
            EXPECT(std::memcmp(got_res.data(), res.data(), res.size() * sizeof(S)) == 0, "mode %d: residual differs from the oracle in the same mode", literal);
            EXPECT(std::memcmp(got_res.data(), res_other.data(), res.size() * sizeof(S)) != 0, "mode %d: residual must differ from the other mode's", literal);
            CHECK(hipFree(d_out)); CHECK(hipFree(d_res)); CHECK(hipFree(d_bias)); CHECK(hipFree(d_gamma));
        }
        {   // QKV: the bias is added by default and ignored in the literal mode
            const int batch = 2, seq = 9, hn = 32, kvn = 32, hs = 128;
            const std::vector<int> lens = {9, 4}, hist = {5, 0};
            const int tokens = 13;
            std::mt19937 gen(22);
            auto qkv = randn<T>((size_t)tokens * (hn + 2 * kvn) * hs, 1.f, gen);
            auto bias = randn<T>((size_t)(hn + 2 * kvn) * hs, 0.5f, gen);
            std::vector<int> po(batch * seq, 0), cum(batch + 1, 0);
            isp_oracle_cal_padding_offset(po.data(), cum.data(), lens.data(), batch, seq);
            int *d_lens = to_device(lens), *d_hist = to_device(hist), *d_po = to_device(po);
            TensorWrapper<int> po_t(Device::GPU, getTensorType<int>(), {batch, seq}, d_po);
            TensorWrapper<int> lens_t(Device::GPU, getTensorType<int>(), {batch}, d_lens);
            TensorWrapper<int> hist_t(Device::GPU, getTensorType<int>(), {batch}, d_hist);
            const size_t qn = (size_t)batch * hn * seq * hs;
            const S sentinel = Host<T>::to(-77.f);
            S *dq = to_device(std::vector<S>(qn, sentinel)), *dk = to_device(std::vector<S>(qn, sentinel)), *dv = to_device(std::vector<S>(qn, sentinel));
            S *d_qkv = to_device(qkv), *d_bias = to_device(bias);
            TensorWrapper<T> q_t(Device::GPU, getTensorType<T>(), {batch, hn, seq, hs}, (T*)dq);
            TensorWrapper<T> k_t(Device::GPU, getTensorType<T>(), {batch, kvn, seq, hs}, (T*)dk);
            TensorWrapper<T> v_t(Device::GPU, getTensorType<T>(), {batch, kvn, seq, hs}, (T*)dv);
            TensorWrapper<T> qkv_t(Device::GPU, getTensorType<T>(), {tokens, hn + 2 * kvn, hs}, (T*)d_qkv);
            BaseWeight<T> w;
            w.bias = (T*)d_bias;
            LLaMAAttentionStaticParams params;
            launchAddFusedQKVBiasTransposeAndRoPE(&q_t, &k_t, &v_t, &qkv_t, w, &po_t, &hist_t, &lens_t, params);
            std::vector<S> eq(qn, sentinel), ek(qn, sentinel), ev(qn, sentinel);
            const void* oracle_bias = literal ? nullptr : bias.data();
            if (std::is_same<T, float>::value)
                isp_oracle_qkv_rope_f32((float*)eq.data(), (float*)ek.data(), (float*)ev.data(), (const float*)qkv.data(), (const float*)oracle_bias,
                                        po.data(), hist.data(), lens.data(), batch, seq, tokens, hn, kvn, hs, 128, 10000.f);
            else
                isp_oracle_qkv_rope_f16((uint16_t*)eq.data(), (uint16_t*)ek.data(), (uint16_t*)ev.data(), (const uint16_t*)qkv.data(),
                                        (const uint16_t*)oracle_bias, po.data(), hist.data(), lens.data(), batch, seq, tokens, hn, kvn, hs, 128, 10000.f);
            auto mag = [](size_t) { return 8.0; };
            compare<T>(to_host(dq, qn), eq, literal ? "literal mode: q" : "default mode: q", mag);
            compare<T>(to_host(dk, qn), ek, literal ? "literal mode: k" : "default mode: k", mag);
            auto gv = to_host(dv, qn);
            EXPECT(std::memcmp(gv.data(), ev.data(), qn * sizeof(S)) == 0, "mode %d: v differs from the oracle in the same mode", literal);
            CHECK(hipFree(dq)); CHECK(hipFree(dk)); CHECK(hipFree(dv)); CHECK(hipFree(d_qkv)); CHECK(hipFree(d_bias));
            CHECK(hipFree(d_lens)); CHECK(hipFree(d_hist)); CHECK(hipFree(d_po));
        }
    }
    isp_shims::setReferenceLiteralBias(before);
}

// --------------------------------------------------------------------------- swiglu
template <typename T>
void case_act() {
    using S = typename Host<T>::Store;
    {  // the reference's own case: all ones, [16, 2, 11008]
        const int batch_size = 16, intermedia_size = 11008;
        S* d_input = to_device(std::vector<S>((size_t)batch_size * 2 * intermedia_size, Host<T>::to(1.f)));
        S* d_output = to_device(std::vector<S>((size_t)batch_size * intermedia_size));
        TensorWrapper<T>* input_tensor = new TensorWrapper<T>(GPU, getTensorType<T>(), {batch_size, 2, intermedia_size}, (T*)d_input);
        TensorWrapper<T>* output_tensor = new TensorWrapper<T>(GPU, getTensorType<T>(), {batch_size, intermedia_size}, (T*)d_output);
        launchAct(input_tensor, output_tensor);
        auto out = to_host(d_output, (size_t)batch_size * intermedia_size);
        const float expect = Host<T>::from(Host<T>::to(0.7310585786300049f));
        for (size_t i = 0; i < out.size(); i++)
            EXPECT(std::fabs(Host<T>::from(out[i]) - expect) <= 1e-6f, "known answer [%zu] = %g", i, Host<T>::from(out[i]));
    }
    const int tokens = 37, inter = 11008;
    std::mt19937 gen(5);
    auto in = randn<T>((size_t)tokens * 2 * inter, 1.5f, gen);
    S* d_in = to_device(in);
    S* d_out = to_device(std::vector<S>((size_t)tokens * inter));
    TensorWrapper<T> in_t(GPU, getTensorType<T>(), {tokens, 2, inter}, (T*)d_in);
    TensorWrapper<T> out_t(GPU, getTensorType<T>(), {tokens, inter}, (T*)d_out);
    launchAct(&in_t, &out_t);
    std::vector<S> ref((size_t)tokens * inter);
    if (std::is_same<T, float>::value) isp_oracle_swiglu_f32((const float*)in.data(), (float*)ref.data(), tokens, inter);
    else isp_oracle_swiglu_f16((const uint16_t*)in.data(), (uint16_t*)ref.data(), tokens, inter);
    // relative to |silu(g)| * |u| with a floor from the inputs (fp32 criterion)
    auto mag = [&](size_t i) { size_t t = i / inter, c = i % inter; return 1e-2 * std::fabs((double)Host<T>::from(in[(t * 2 + 1) * inter + c])); };
    compare<T>(to_host(d_out, ref.size()), ref, "swiglu", std::is_same<T, float>::value ? std::function<double(size_t)>(mag) : nullptr);
}

// --------------------------------------------------------------------------- error behaviour
void case_errors() {
    int* d_i = to_device(std::vector<int>(64, 0));
    float* d_f = to_device(std::vector<float>(4096, 0.f));
    TensorWrapper<int> ids(GPU, INT32, {5}, d_i);
    TensorWrapper<float> out(GPU, FP32, {4, 8}, d_f);
    EmbeddingWeight<float> table;
    table.data = d_f;
    EXPECT(throws([&] { launchInputEmbedding(&ids, &out, &table); }), "embedding: token count mismatch must throw");
    TensorWrapper<float> bad_act(GPU, FP32, {4, 3, 8}, d_f);
    EXPECT(throws([&] { launchAct(&bad_act, &out); }), "act: shape[1] != 2 must throw");
    TensorWrapper<int> po(GPU, INT32, {3, 5}, d_i), cum(GPU, INT32, {3}, d_i), lens(GPU, INT32, {3}, d_i), lens2(GPU, INT32, {2}, d_i);
    EXPECT(throws([&] { launchCalPaddingoffset(&po, &cum, &lens); }), "padding: cum_seqlens size must throw");
    TensorWrapper<int> cum4(GPU, INT32, {4}, d_i);
    EXPECT(throws([&] { launchCalPaddingoffset(&po, &cum4, &lens2); }), "padding: lengths size must throw");
    EXPECT(throws([&] { TensorWrapper<float> wrong(GPU, FP16, {1}, d_f); }), "dtype mismatch in the TensorWrapper ctor must throw");
    EXPECT(throws([&] { (void)ids.getVal(); }), "getVal on a GPU tensor must throw");
    TensorWrapper<float> null_out(GPU, FP32, {4, 8}, nullptr);
    LayerNormWeight<float> w;
    w.gamma = d_f;
    EXPECT(throws([&] { launchRMSNorm(&null_out, w, 1e-5f); }), "null data must throw, not fault");
    EXPECT(null_out.size() == 0 && out.size() == 32, "size()");
    TensorMap m({{"out", &out}});
    EXPECT(m.isExist("out") && m.at("out") == &out && m.size() == 1, "TensorMap");
    EXPECT(throws([&] { TensorMap bad({{"null", &null_out}}); }), "TensorMap must reject tensors without storage");
}

int main(int argc, char** argv) {
    const std::string which = argc > 1 ? argv[1] : "all";
    std::map<std::string, std::function<void()>> cases = {
        {"embedding", [] { case_embedding<half>(); case_embedding<float>(); }},
        {"padding", [] { case_padding(); }},
        {"norm", [] { case_norm<float>(); case_norm<half>(); }},
        {"rmsnorm", [] { case_rmsnorm<float>(); case_rmsnorm<half>(); }},
        {"qkv", [] { case_qkv<float>(); case_qkv<half>(); }},
        {"act", [] { case_act<float>(); case_act<half>(); }},
        {"bias_modes", [] { case_bias_modes<float>(); case_bias_modes<half>(); }},
        {"errors", [] { case_errors(); }},
    };
    for (auto& kv : cases) {
        if (which != "all" && which != kv.first) continue;
        std::printf("[case] %s\n", kv.first.c_str());
        std::fflush(stdout);
        kv.second();
        CHECK(hipDeviceSynchronize());
    }
    if (g_failures) {
        std::printf("%d check(s) failed\n", g_failures);
        return 1;
    }
    std::printf("passed\n");
    return 0;
}
