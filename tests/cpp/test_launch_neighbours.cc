// Reference-style call sites for the launchers either side of the fused QKV step: launchRoPE (decode),
// launchTransposeOutRemovePadding, launchConcatKVCache, launchRepeatKVCache -- TensorWrapper arguments
// built as the reference's tests/unittests programs build them, results checked against the CPU oracle.
//
//   test_launch_neighbours <case>      case = rope | transpose | kvcache | all
#include <map>

#include "src/kernels/concat_past_kv.h"
#include "src/kernels/fused_transpose_and_remv_pad.h"
#include "src/kernels/qkv_bias_and_RoPE.h"
#include "src/kernels/repeat_kv.h"
#include "test_util.h"

template <typename T>
void case_rope() {
    using S = typename Host<T>::Store;
    const int head_num = 32, head_size = 128, qkv_heads = 96;
    std::mt19937 gen(11);
    auto x = randn<T>((size_t)qkv_heads * head_size, 1.f, gen);
    S* d_x = to_device(x);
    TensorWrapper<T> qkv_buf(Device::GPU, getTensorType<T>(), {1, qkv_heads, head_size}, (T*)d_x);
    int cur_step = 23;
    TensorWrapper<int> step(Device::CPU, getTensorType<int>(), {1}, &cur_step);  // host tensor, read with getVal()
    LLaMAAttentionStaticParams params;
    launchRoPE(&qkv_buf, &step, params);
    auto got = to_host(d_x, x.size());
    if (std::is_same<T, float>::value) isp_oracle_rope_decode_f32((float*)x.data(), 1, head_num, head_num, head_size, cur_step, 128, 10000.f);
    else isp_oracle_rope_decode_f16((uint16_t*)x.data(), 1, head_num, head_num, head_size, cur_step, 128, 10000.f);
    compare<T>(got, x, "decode rope", [](size_t) { return 6.0; });
    EXPECT(std::memcmp(got.data() + 64 * head_size, x.data() + 64 * head_size, 32 * head_size * sizeof(S)) == 0, "v heads changed");
    // the reference's shape checks
    TensorWrapper<T> two_rows(Device::GPU, getTensorType<T>(), {2, qkv_heads, head_size}, (T*)d_x);
    EXPECT(throws([&] { launchRoPE(&two_rows, &step, params); }), "batch != 1 must throw");
    TensorWrapper<int> gpu_step(Device::GPU, getTensorType<int>(), {1}, &cur_step);
    EXPECT(throws([&] { launchRoPE(&qkv_buf, &gpu_step, params); }), "a GPU-resident step tensor must throw (getVal)");
}

template <typename T>
void case_transpose() {
    using S = typename Host<T>::Store;
    {  // the reference's example
        const int batch_size = 2, head_num = 2, max_seq_len = 4, head_size = 2, num_tokens = 5;
        std::vector<S> h_in(batch_size * head_num * max_seq_len * head_size);
        for (size_t i = 0; i < h_in.size(); i++) h_in[i] = Host<T>::to((float)i);
        std::vector<int> h_padding_offset = {0, 0, 2, 2, 2};
        S* d_in = to_device(h_in);
        S* d_out = to_device(std::vector<S>(num_tokens * head_num * head_size));
        int* d_padding_offset = to_device(h_padding_offset);
        TensorWrapper<T>* in = new TensorWrapper<T>(Device::GPU, getTensorType<T>(), {batch_size, head_num, max_seq_len, head_size}, (T*)d_in);
        TensorWrapper<int>* in_pad = new TensorWrapper<int>(Device::GPU, getTensorType<int>(), {num_tokens}, d_padding_offset);
        TensorWrapper<T>* out = new TensorWrapper<T>(Device::GPU, getTensorType<T>(), {num_tokens, head_num, head_size}, (T*)d_out);
        launchTransposeOutRemovePadding(in, in_pad, out);
        auto h_out = to_host(d_out, num_tokens * head_num * head_size);
        const float expect[20] = {0, 1, 8, 9, 2, 3, 10, 11, 16, 17, 24, 25, 18, 19, 26, 27, 20, 21, 28, 29};
        for (int i = 0; i < 20; i++) EXPECT(Host<T>::from(h_out[i]) == expect[i], "out[%d] = %g", i, Host<T>::from(h_out[i]));
    }
    const int batch = 4, heads = 32, seq = 48, hs = 128;
    const std::vector<int> lens = {48, 5, 31, 1};
    int tokens = 0;
    for (int l : lens) tokens += l;
    std::vector<int> po(batch * seq, 0), cum(batch + 1, 0);
    isp_oracle_cal_padding_offset(po.data(), cum.data(), lens.data(), batch, seq);
    std::mt19937 gen(12);
    auto src = randn<T>((size_t)batch * heads * seq * hs, 1.f, gen);
    S* d_src = to_device(src);
    S* d_dst = to_device(std::vector<S>((size_t)tokens * heads * hs));
    int* d_po = to_device(po);
    TensorWrapper<T> in(Device::GPU, getTensorType<T>(), {batch, heads, seq, hs}, (T*)d_src);
    TensorWrapper<int> pad(Device::GPU, getTensorType<int>(), {tokens}, d_po);
    TensorWrapper<T> out(Device::GPU, getTensorType<T>(), {tokens, heads, hs}, (T*)d_dst);
    launchTransposeOutRemovePadding(&in, &pad, &out);
    std::vector<S> ref((size_t)tokens * heads * hs);
    isp_oracle_transpose_remove_padding(src.data(), ref.data(), po.data(), batch, heads, seq, hs, tokens, sizeof(S));
    auto got = to_host(d_dst, ref.size());
    EXPECT(std::memcmp(got.data(), ref.data(), ref.size() * sizeof(S)) == 0, "transpose-remove-padding differs from the oracle");
}

template <typename T>
void case_kvcache() {
    using S = typename Host<T>::Store;
    const int layers = 2, batch = 2, kv_heads = 4, heads = 8, max_q = 6, max_seq = 20, hs = 128;
    std::mt19937 gen(13);
    auto k_src = randn<T>((size_t)batch * kv_heads * max_q * hs, 1.f, gen);
    auto v_src = randn<T>((size_t)batch * kv_heads * max_q * hs, 1.f, gen);
    auto k_cache = randn<T>((size_t)layers * batch * kv_heads * max_seq * hs, 1.f, gen);
    auto v_cache = randn<T>((size_t)layers * batch * kv_heads * max_seq * hs, 1.f, gen);
    const std::vector<int> cur = {6, 2}, hist = {3, 11};
    int layer = 1;
    S *d_ks = to_device(k_src), *d_vs = to_device(v_src), *d_kc = to_device(k_cache), *d_vc = to_device(v_cache);
    int *d_cur = to_device(cur), *d_hist = to_device(hist);
    TensorWrapper<T> ks(Device::GPU, getTensorType<T>(), {batch, kv_heads, max_q, hs}, (T*)d_ks);
    TensorWrapper<T> vs(Device::GPU, getTensorType<T>(), {batch, kv_heads, max_q, hs}, (T*)d_vs);
    TensorWrapper<T> kc(Device::GPU, getTensorType<T>(), {layers, batch, kv_heads, max_seq, hs}, (T*)d_kc);
    TensorWrapper<T> vc(Device::GPU, getTensorType<T>(), {layers, batch, kv_heads, max_seq, hs}, (T*)d_vc);
    TensorWrapper<int> layer_id(Device::CPU, getTensorType<int>(), {1}, &layer);
    TensorWrapper<int> cur_t(Device::GPU, getTensorType<int>(), {batch}, d_cur);
    TensorWrapper<int> hist_t(Device::GPU, getTensorType<int>(), {batch}, d_hist);
    launchConcatKVCache(&ks, &vs, &layer_id, &cur_t, &hist_t, &kc, &vc);
    const size_t layer_off = (size_t)layer * batch * kv_heads * max_seq * hs;
    isp_oracle_concat_kv(k_src.data(), k_cache.data(), layer_off, cur.data(), hist.data(), batch, kv_heads, max_q, max_seq, hs, sizeof(S));
    isp_oracle_concat_kv(v_src.data(), v_cache.data(), layer_off, cur.data(), hist.data(), batch, kv_heads, max_q, max_seq, hs, sizeof(S));
    auto gk = to_host(d_kc, k_cache.size()), gv = to_host(d_vc, v_cache.size());
    EXPECT(std::memcmp(gk.data(), k_cache.data(), k_cache.size() * sizeof(S)) == 0, "k cache differs from the oracle");
    EXPECT(std::memcmp(gv.data(), v_cache.data(), v_cache.size() * sizeof(S)) == 0, "v cache differs from the oracle");

    const std::vector<int> ctx = {9, 13};
    const int max_k = 13;
    const S fill = Host<T>::to(-3.f);
    S* d_kd = to_device(std::vector<S>((size_t)batch * heads * max_k * hs, fill));
    S* d_vd = to_device(std::vector<S>((size_t)batch * heads * max_k * hs, fill));
    int* d_ctx = to_device(ctx);
    TensorWrapper<int> ctx_t(Device::GPU, getTensorType<int>(), {batch}, d_ctx);
    TensorWrapper<T> kd(Device::GPU, getTensorType<T>(), {batch, heads, max_k, hs}, (T*)d_kd);
    TensorWrapper<T> vd(Device::GPU, getTensorType<T>(), {batch, heads, max_k, hs}, (T*)d_vd);
    launchRepeatKVCache(&kc, &vc, &ctx_t, &layer_id, &kd, &vd);
    std::vector<S> ek((size_t)batch * heads * max_k * hs, fill), ev(ek);
    isp_oracle_repeat_kv(k_cache.data(), ek.data(), layer_off, ctx.data(), batch, heads, kv_heads, max_seq, max_k, hs, sizeof(S));
    isp_oracle_repeat_kv(v_cache.data(), ev.data(), layer_off, ctx.data(), batch, heads, kv_heads, max_seq, max_k, hs, sizeof(S));
    auto rk = to_host(d_kd, ek.size()), rv = to_host(d_vd, ev.size());
    EXPECT(std::memcmp(rk.data(), ek.data(), ek.size() * sizeof(S)) == 0, "repeated k differs from the oracle");
    EXPECT(std::memcmp(rv.data(), ev.data(), ev.size() * sizeof(S)) == 0, "repeated v differs from the oracle");
}

int main(int argc, char** argv) {
    const std::string which = argc > 1 ? argv[1] : "all";
    std::map<std::string, std::function<void()>> cases = {
        {"rope", [] { case_rope<float>(); case_rope<half>(); }},
        {"transpose", [] { case_transpose<float>(); case_transpose<half>(); }},
        {"kvcache", [] { case_kvcache<float>(); case_kvcache<half>(); }},
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
