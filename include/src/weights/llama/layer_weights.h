// Weights of one LLaMA decoder layer, with the reference's class name, constructor and public members
// (src/weights/llama/layer_weights.h:6-36).  The constructor allocates device memory in the shapes
// the reference declares (src/weights/llama/layer_weights.cc:19-41) -- every matrix row-major
// [out_features, in_features]:
//   self_attn_weight.qkv     [(head_num + 2 kv_head_num) * head_size, hidden]
//   self_attn_weight.output  [hidden, hidden]
//   ffn_weight.gateAndup     [2 * inter_size, hidden]
//   ffn_weight.down          [hidden, inter_size]
// and the optional biases when attn_bias is set.  loadWeights() fills them with small deterministic
// values ("dummy" weights, as the reference's no-argument loadWeights does for performance runs).
// loadWeights(weight_path, weight_type) reads the per-tensor files the reference's converter writes
// (src/weights/llama/layer_weights.cc:45-62: raw little-endian fp32, `weight_path` + ".input_layernorm.weight.bin",
// ".post_attention_layernorm.weight.bin", ".self_attn.qkv.weight.bin", ".self_attn.o_proj.weight.bin",
// ".mlp.gate_up_proj.weight.bin", ".mlp.down_proj.weight.bin", and with attn_bias ".attention.wqkv.bias.bin",
// ".attention.wo.bias.bin"), converts to T and uploads; without attn_bias the three biases are set to nullptr as
// the reference does.  One difference: a file that is missing or shorter than its declared shape throws
// std::runtime_error (the reference's helper prints a message and leaves the tensor as it was).
#pragma once
#include <string>

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
    int bit_size;
    bool attn_bias;

public:
    LlamaLayerWeight() = delete;
    LlamaLayerWeight(int head_num, int kv_head_num, int head_size, int inter_size, WeightType weight_type,
                     bool attn_bias);
    LlamaLayerWeight(const LlamaLayerWeight&) = delete;
    LlamaLayerWeight& operator=(const LlamaLayerWeight&) = delete;
    ~LlamaLayerWeight();

    void loadWeights(std::string weight_path, WeightType weight_type);

    void loadWeights();

    LayerNormWeight<T> attn_norm_weight;
    LayerNormWeight<T> ffn_norm_weight;
    LLaMAattentionWeights<T> self_attn_weight;
    LLaMAFFNWeights<T> ffn_weight;
};
