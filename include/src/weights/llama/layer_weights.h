// Weights of one LLaMA decoder layer, with the reference's class name, constructor and public members
// (src/weights/llama/layer_weights.h:6-36).  The constructor allocates device memory in the shapes
// the reference declares (src/weights/llama/layer_weights.cc:19-41) -- every matrix row-major
// [out_features, in_features]:
//   self_attn_weight.qkv     [(head_num + 2 kv_head_num) * head_size, hidden]
//   self_attn_weight.output  [hidden, hidden]
//   ffn_weight.gateAndup     [2 * inter_size, hidden]
//   ffn_weight.down          [hidden, inter_size]
// and the optional biases when attn_bias is set.  loadWeights() fills them with small deterministic
// values ("dummy" weights, as the reference's no-argument loadWeights does for performance runs);
// loading from checkpoint files is outside this library (the reference's loader lives in
// src/utils/weight_utils.cu).
#pragma once
#include "src/weights/llama/attention_weights.h"
#include "src/weights/llama/ffn_weights.h"
#include "src/weights/llama/norm_weights.h"

template <typename T>
class LlamaLayerWeight {
private:
    int head_num;
    int kv_head_num;
    int head_size;
    int hidden_units;
    int inter_size;
    WeightType weight_type;
    bool attn_bias;

public:
    LlamaLayerWeight() = delete;
    LlamaLayerWeight(int head_num, int kv_head_num, int head_size, int inter_size, WeightType weight_type,
                     bool attn_bias);
    LlamaLayerWeight(const LlamaLayerWeight&) = delete;
    LlamaLayerWeight& operator=(const LlamaLayerWeight&) = delete;
    ~LlamaLayerWeight();

    void loadWeights();

    LayerNormWeight<T> attn_norm_weight;
    LayerNormWeight<T> ffn_norm_weight;
    LLaMAattentionWeights<T> self_attn_weight;
    LLaMAFFNWeights<T> ffn_weight;
};
