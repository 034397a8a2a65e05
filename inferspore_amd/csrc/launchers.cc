// The reference's C++ launch* entry points, as thin shims over the C ABI (inferspore_amd.h).
// Each shim unpacks shapes and pointers from the TensorWrapper / weight structs the way the
// reference's launcher does (cited per function), keeps the reference's own argument checks, and
// launches on the null stream like the reference.  A non-zero status from the C ABI becomes the
// same std::runtime_error the reference's LLM_CHECK raises.
#include <atomic>
#include <cstdlib>
#include <cstring>

#include "inferspore_amd.h"
#include "inferspore_amd_shims.h"
#include "src/kernels/act_kernel.h"
#include "src/kernels/cal_paddingoffset.h"
#include "src/kernels/concat_past_kv.h"
#include "src/kernels/fused_addresidual_norm.h"
#include "src/kernels/fused_transpose_and_remv_pad.h"
#include "src/kernels/input_embedding.h"
#include "src/kernels/qkv_bias_and_RoPE.h"
#include "src/kernels/repeat_kv.h"
#include "src/kernels/rmsnorm.h"

namespace {

template <typename T>
struct Abi;
template <>
struct Abi<float> {
    static constexpr auto embedding = isp_embedding_f32;
    static constexpr auto rmsnorm = isp_rmsnorm_f32;
    static constexpr auto fused_norm = isp_fused_add_bias_residual_rmsnorm_f32;
    static constexpr auto qkv = isp_qkv_bias_rope_transpose_f32;
    static constexpr auto qkv_append = isp_qkv_bias_rope_transpose_append_f32;
    static constexpr auto swiglu = isp_swiglu_f32;
    static constexpr auto rope_decode = isp_rope_decode_f32;
    static constexpr auto transpose_remove_padding = isp_transpose_remove_padding_f32;
    static constexpr auto concat_kv = isp_concat_kv_cache_f32;
    static constexpr auto repeat_kv = isp_repeat_kv_cache_f32;
};
template <>
struct Abi<half> {
    static constexpr auto embedding = isp_embedding_f16;
    static constexpr auto rmsnorm = isp_rmsnorm_f16;
    static constexpr auto fused_norm = isp_fused_add_bias_residual_rmsnorm_f16;
    static constexpr auto qkv = isp_qkv_bias_rope_transpose_f16;
    static constexpr auto qkv_append = isp_qkv_bias_rope_transpose_append_f16;
    static constexpr auto swiglu = isp_swiglu_f16;
    static constexpr auto rope_decode = isp_rope_decode_f16;
    static constexpr auto transpose_remove_padding = isp_transpose_remove_padding_f16;
    static constexpr auto concat_kv = isp_concat_kv_cache_f16;
    static constexpr auto repeat_kv = isp_repeat_kv_cache_f16;
};

std::atomic<int>& literal_bias_setting() {
    static std::atomic<int> setting([] {
        const char* env = std::getenv("ISP_SHIMS_REFERENCE_LITERAL_BIAS");
        return (env != nullptr && std::strcmp(env, "1") == 0) ? 1 : 0;
    }());
    return setting;
}

inline void expect_ok(int status, const char* what) {
    LLM_CHECK_WITH_INFO(status == ISP_OK, std::string(what) + ": " + isp_strerror(status));
}

}  // namespace

namespace isp_shims {
bool setReferenceLiteralBias(bool on) { return literal_bias_setting().exchange(on ? 1 : 0) != 0; }
bool referenceLiteralBias() { return literal_bias_setting().load() != 0; }
}  // namespace isp_shims

// reference: src/kernels/input_embedding.cu:25-45 (token count and hidden size from output->shape,
// the shape check at :35)
template <typename T>
void launchInputEmbedding(TensorWrapper<int>* input_ids, TensorWrapper<T>* output,
                          EmbeddingWeight<T>* embed_table) {
    const int tokens = output->shape[0];
    const int hidden = output->shape[1];
    LLM_CHECK_WITH_INFO(tokens == input_ids->shape[0],
                        "input ids 1st shape should equal to 1st shape of output");
    const int vocab = embed_table->shape.size() == 2 ? embed_table->shape[0] : 0;
    expect_ok(Abi<T>::embedding(input_ids->data, output->data, embed_table->data, tokens, hidden,
                                vocab, nullptr),
              "launchInputEmbedding");
}

// reference: src/kernels/cal_paddingoffset.cu:49-60
void launchCalPaddingoffset(TensorWrapper<int>* padding_offset, TensorWrapper<int>* cum_seqlens,
                            TensorWrapper<int>* input_lengths) {
    const int batch = padding_offset->shape[0];
    const int max_q_len = padding_offset->shape[1];
    LLM_CHECK_WITH_INFO(batch == input_lengths->shape[0],
                        "input lenghts numbers should equal to padding offset bs dim!");
    LLM_CHECK_WITH_INFO(batch == cum_seqlens->shape[0] - 1,
                        "cum seqlen numbers should equal to padding offset bs dim + 1!");
    expect_ok(isp_cal_padding_offset(padding_offset->data, cum_seqlens->data, input_lengths->data,
                                     batch, max_q_len, nullptr),
              "launchCalPaddingoffset");
}

// reference: src/kernels/fused_addresidual_norm.cu:143-170 (tokens, hidden from decoder_out->shape;
// bias = norm.bias; gamma = scale)
template <typename T>
void launchFusedAddBiasResidualRMSNorm(TensorWrapper<T>* residual, TensorWrapper<T>* decoder_out,
                                       BaseWeight<T>& norm, T* scale, float eps) {
    const int tokens = decoder_out->shape[0];
    const int hidden = decoder_out->shape[1];
    const unsigned flags = isp_shims::referenceLiteralBias() ? ISP_NORM_RESIDUAL_EXCLUDES_BIAS : 0u;
    expect_ok(Abi<T>::fused_norm(residual->data, decoder_out->data, norm.bias, scale, eps, tokens,
                                 hidden, flags, nullptr),
              "launchFusedAddBiasResidualRMSNorm");
}

template <typename T>
void launchRMSNorm(TensorWrapper<T>* decoder_out, LayerNormWeight<T>& norm, float eps) {
    expect_ok(Abi<T>::rmsnorm(decoder_out->data, norm.gamma, eps, decoder_out->shape[0],
                              decoder_out->shape[1], nullptr),
              "launchRMSNorm");
}

// reference: src/kernels/qkv_bias_and_RoPE.cu:286-330 (shape derivation :298-304)
template <typename T>
void launchAddFusedQKVBiasTransposeAndRoPE(TensorWrapper<T>* q_buf, TensorWrapper<T>* k_buf,
                                           TensorWrapper<T>* v_buf, TensorWrapper<T>* QKV,
                                           BaseWeight<T>& qkv, TensorWrapper<int>* padding_offset,
                                           TensorWrapper<int>* history_length,
                                           TensorWrapper<int>* input_length,
                                           LLaMAAttentionStaticParams& params) {
    const int token_num = QKV->shape[0];
    const int qkv_head_num = QKV->shape[1];
    const int head_size = QKV->shape[2];
    const int batch_size = q_buf->shape[0];
    const int head_num = q_buf->shape[1];
    const int seq_len = q_buf->shape[2];
    const int kv_head_num = (qkv_head_num - head_num) / 2;
    const T* bias = isp_shims::referenceLiteralBias() ? nullptr : qkv.bias;
    expect_ok(Abi<T>::qkv(q_buf->data, k_buf->data, v_buf->data, QKV->data, bias,
                          padding_offset->data, history_length->data, input_length->data,
                          batch_size, seq_len, token_num, head_num, kv_head_num, head_size,
                          params.rotary_embedding_dim, params.rotary_embedding_base,
                          params.max_position_embeddings, params.use_dynamic_ntk ? 1 : 0, nullptr),
              "launchAddFusedQKVBiasTransposeAndRoPE");
}

// shapes as above; kv_head_num and max_seq_len from the cache [layers, batch, kv_head_num, max_seq_len, hs]
template <typename T>
void launchAddFusedQKVBiasTransposeRoPEAndConcatKV(TensorWrapper<T>* q_buf, TensorWrapper<T>* QKV,
                                                   BaseWeight<T>& qkv,
                                                   TensorWrapper<int>* padding_offset,
                                                   TensorWrapper<int>* history_length,
                                                   TensorWrapper<int>* input_length,
                                                   TensorWrapper<int>* layer_id,
                                                   TensorWrapper<T>* k_cache,
                                                   TensorWrapper<T>* v_cache,
                                                   LLaMAAttentionStaticParams& params) {
    const int token_num = QKV->shape[0];
    const int qkv_head_num = QKV->shape[1];
    const int head_size = QKV->shape[2];
    const int batch_size = q_buf->shape[0];
    const int head_num = q_buf->shape[1];
    const int seq_len = q_buf->shape[2];
    const int kv_head_num = (qkv_head_num - head_num) / 2;
    LLM_CHECK_WITH_INFO(k_cache->shape.size() == 5 && k_cache->shape == v_cache->shape,
                        "k / v cache should be [layers, batch, kv heads, max seq len, head size]");
    LLM_CHECK_WITH_INFO(k_cache->shape[1] == batch_size && k_cache->shape[2] == kv_head_num &&
                            k_cache->shape[4] == head_size,
                        "k / v cache extents should match the qkv buffer's");
    const int layer = layer_id->getVal();
    LLM_CHECK_WITH_INFO(layer >= 0 && layer < k_cache->shape[0], "layer id outside the cache");
    const T* bias = isp_shims::referenceLiteralBias() ? nullptr : qkv.bias;
    expect_ok(Abi<T>::qkv_append(q_buf->data, nullptr, nullptr, k_cache->data, v_cache->data, layer,
                                 k_cache->shape[3], QKV->data, bias, padding_offset->data,
                                 history_length->data, input_length->data, batch_size, seq_len,
                                 token_num, head_num, kv_head_num, head_size,
                                 params.rotary_embedding_dim, params.rotary_embedding_base, nullptr),
              "launchAddFusedQKVBiasTransposeRoPEAndConcatKV");
}

// reference: src/kernels/act_kernel.cu:57-71 (the shape[1] == 2 check at :61)
template <typename T>
void launchAct(TensorWrapper<T>* input, TensorWrapper<T>* out) {
    const int tokens = input->shape[0];
    LLM_CHECK(input->shape[1] == 2);
    const int inter = input->shape[2];
    expect_ok(Abi<T>::swiglu(input->data, out->data, tokens, inter, nullptr), "launchAct");
}

// reference: src/kernels/qkv_bias_and_RoPE.cu:404-434 (hard-wired to LLaMA-7B: 32 q heads, batch 1)
template <typename T>
void launchRoPE(TensorWrapper<T>* qkv_buf, TensorWrapper<int>* step,
                LLaMAAttentionStaticParams& static_params) {
    const int batch_size = qkv_buf->shape[0];
    const int qkv_head_num = qkv_buf->shape[1];
    const int head_num = 32;
    const int head_size = qkv_buf->shape[2];
    LLM_CHECK(batch_size == 1);
    LLM_CHECK(qkv_head_num == 96);
    LLM_CHECK(head_size == 128);
    const int cur_step = step->getVal();
    expect_ok(Abi<T>::rope_decode(qkv_buf->data, batch_size, head_num, head_num, head_size, cur_step,
                                  static_params.rotary_embedding_dim,
                                  static_params.rotary_embedding_base, nullptr),
              "launchRoPE");
}

// contract: src/kernels/fused_transpose_and_remv_pad.h:7-10, tests/unittests/test_fused_trans_remv_pad.cu:40-49
template <typename T>
void launchTransposeOutRemovePadding(TensorWrapper<T>* qkv_buf_w_pad, TensorWrapper<int>* padding_offset,
                                     TensorWrapper<T>* qkv_buf_wo_pad_1) {
    const int batch_size = qkv_buf_w_pad->shape[0];
    const int head_num = qkv_buf_w_pad->shape[1];
    const int seq_len = qkv_buf_w_pad->shape[2];
    const int head_size = qkv_buf_w_pad->shape[3];
    const int token_num = qkv_buf_wo_pad_1->shape[0];
    expect_ok(Abi<T>::transpose_remove_padding(qkv_buf_w_pad->data, padding_offset->data,
                                               qkv_buf_wo_pad_1->data, batch_size, head_num, seq_len,
                                               head_size, token_num, nullptr),
              "launchTransposeOutRemovePadding");
}

// reference: src/kernels/concat_past_kv.cu:76-113 (shape derivation :84-90)
template <typename T>
void launchConcatKVCache(TensorWrapper<T>* k_src, TensorWrapper<T>* v_src, TensorWrapper<int>* layer_id,
                         TensorWrapper<int>* cur_query_length, TensorWrapper<int>* history_length,
                         TensorWrapper<T>* k_dst, TensorWrapper<T>* v_dst) {
    const int batch_size = k_src->shape[0];
    const int max_seq_len = k_dst->shape[3];
    const int kv_head_num = k_src->shape[1];
    const int max_q_len = k_src->shape[2];
    const int head_size = k_src->shape[3];
    const int layer = layer_id->getVal();
    expect_ok(Abi<T>::concat_kv(k_src->data, v_src->data, k_dst->data, v_dst->data, layer,
                                cur_query_length->data, history_length->data, batch_size, kv_head_num,
                                max_q_len, max_seq_len, head_size, nullptr),
              "launchConcatKVCache");
}

// reference: src/kernels/repeat_kv.cu:52-100 (shape derivation :59-70)
template <typename T>
void launchRepeatKVCache(TensorWrapper<T>* k_cache_src, TensorWrapper<T>* v_cache_src,
                         TensorWrapper<int>* context_length, TensorWrapper<int>* layer_id,
                         TensorWrapper<T>* k_cache_dst, TensorWrapper<T>* v_cache_dst) {
    const int batch_size = context_length->shape[0];
    const int kv_head_num = k_cache_src->shape[2];
    const int max_seq_len = k_cache_src->shape[3];
    const int head_num = k_cache_dst->shape[1];
    const int max_k_len = k_cache_dst->shape[2];
    const int head_size = k_cache_dst->shape[3];
    const int layer = layer_id->getVal();
    expect_ok(Abi<T>::repeat_kv(k_cache_src->data, v_cache_src->data, k_cache_dst->data,
                                v_cache_dst->data, layer, context_length->data, batch_size, head_num,
                                kv_head_num, max_seq_len, max_k_len, head_size, nullptr),
              "launchRepeatKVCache");
}

// explicit instantiations for float and half, as in the reference
#define ISP_INSTANTIATE(T)                                                                          \
    template void launchInputEmbedding(TensorWrapper<int>*, TensorWrapper<T>*, EmbeddingWeight<T>*); \
    template void launchFusedAddBiasResidualRMSNorm(TensorWrapper<T>*, TensorWrapper<T>*,           \
                                                    BaseWeight<T>&, T*, float);                     \
    template void launchRMSNorm(TensorWrapper<T>*, LayerNormWeight<T>&, float);                     \
    template void launchAddFusedQKVBiasTransposeAndRoPE(                                            \
        TensorWrapper<T>*, TensorWrapper<T>*, TensorWrapper<T>*, TensorWrapper<T>*, BaseWeight<T>&, \
        TensorWrapper<int>*, TensorWrapper<int>*, TensorWrapper<int>*, LLaMAAttentionStaticParams&); \
    template void launchAddFusedQKVBiasTransposeRoPEAndConcatKV(                                    \
        TensorWrapper<T>*, TensorWrapper<T>*, BaseWeight<T>&, TensorWrapper<int>*,                  \
        TensorWrapper<int>*, TensorWrapper<int>*, TensorWrapper<int>*, TensorWrapper<T>*,           \
        TensorWrapper<T>*, LLaMAAttentionStaticParams&);                                            \
    template void launchAct(TensorWrapper<T>*, TensorWrapper<T>*);                                  \
    template void launchRoPE(TensorWrapper<T>*, TensorWrapper<int>*, LLaMAAttentionStaticParams&);  \
    template void launchTransposeOutRemovePadding(TensorWrapper<T>*, TensorWrapper<int>*,           \
                                                  TensorWrapper<T>*);                               \
    template void launchConcatKVCache(TensorWrapper<T>*, TensorWrapper<T>*, TensorWrapper<int>*,    \
                                      TensorWrapper<int>*, TensorWrapper<int>*, TensorWrapper<T>*,  \
                                      TensorWrapper<T>*);                                           \
    template void launchRepeatKVCache(TensorWrapper<T>*, TensorWrapper<T>*, TensorWrapper<int>*,    \
                                      TensorWrapper<int>*, TensorWrapper<T>*, TensorWrapper<T>*);
ISP_INSTANTIATE(float)
ISP_INSTANTIATE(half)
#undef ISP_INSTANTIATE
