// The stack of context-decoder (prefill) layers: what the reference's model class would call once per
// prompt batch (its factory constructs an absent Llama<T>, src/utils/model_utils.h:40; the per-layer
// weights are the vector the reference's LlamaWeight<T> holds, src/weights/llama/llama_weights.h:13-20).
//
//   padding_offset, cum_seqlens = launchCalPaddingoffset(input_length)
//   residual = decoder_input ; x = launchRMSNorm(decoder_input, layer 0's attn_norm)
//   for every layer l:   x = LlamaContextDecoderLayer::forward(x, residual, weights[l],
//                                next norm = layer l+1's attn_norm, or the model's final norm after the last)
//
// so the result is the final-normed hidden state of every token, ready for the LM head, and the KV cache
// of every layer holds the batch's keys and values.  One layer object serves all layers (its intermediate
// buffers are reused); everything runs on the null stream.
//
// forward() tensors:
//   inputs   "decoder_input"    T   [num_tokens, hidden]   the embedded tokens (launchInputEmbedding); left unchanged
//            "history_length", "input_length", "context_length"   int [batch]   (device)
//   outputs  "decoder_output"   T   [num_tokens, hidden]
//            "all_k_cache", "all_v_cache"   T [layers, batch, kv_head_num, max_seq_len, head_size]
#pragma once
#include <memory>
#include <vector>

#include "src/layers/decoder/context_decoder_layer.h"

template <typename T>
class LlamaContextDecoder {
public:
    LlamaContextDecoder(int head_num, int kv_head_num, int head_size, int inter_size, int num_layers,
                        const LLaMAAttentionStaticParams& attn_params, float rmsnorm_eps, BaseAllocator* allocator);
    ~LlamaContextDecoder();
    LlamaContextDecoder(const LlamaContextDecoder&) = delete;
    LlamaContextDecoder& operator=(const LlamaContextDecoder&) = delete;

    void allocForForward(const LLaMAAttentionDynParams& dyn);
    void freeBuf();

    void forward(TensorMap& inputs, const std::vector<LlamaLayerWeight<T>*>& layer_weights,
                 LayerNormWeight<T>& final_norm, TensorMap& outputs, const LLaMAAttentionDynParams& dyn);

private:
    int num_layers_, hidden_;
    float eps_;
    BaseAllocator* allocator_;
    std::unique_ptr<LlamaContextDecoderLayer<T>> layer_;

    LLaMAAttentionDynParams allocated_;
    int* padding_offset_ = nullptr;  // [batch, max_q_len]
    int* cum_seqlens_ = nullptr;     // [batch + 1]
    T* residual_ = nullptr;          // [tokens, hidden]
    T* hidden_a_ = nullptr;          // [tokens, hidden]  layer input / output, alternating
    T* hidden_b_ = nullptr;
};
