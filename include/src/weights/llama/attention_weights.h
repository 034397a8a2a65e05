// Attention projection weights of one LLaMA layer.
//
// Member names follow the reference's src/weights/llama/attention_weights.h so that code written
// against it (for example its test for the fused QKV step, which passes `attn_weights.qkv`) compiles
// unchanged.  What the kernels of this library read from it:
//   qkv.bias   optional bias of the fused QKV projection, laid out as the packed QKV row is:
//              [head_num * head_size | kv_head_num * head_size | kv_head_num * head_size];
//              nullptr (the default) means "no bias", which is the case for LLaMA checkpoints.
// The weight matrices themselves (q, k, v, qkv, output `.data`) are consumed by GEMMs, which are not
// part of this library.
#pragma once
#include "src/weights/base_weights.h"

template <typename T>
struct LLaMAattentionWeights {
    BaseWeight<T> q;       // separate projections (unused when the fused qkv weight is loaded)
    BaseWeight<T> k;
    BaseWeight<T> v;
    BaseWeight<T> qkv;     // fused [hidden, (head_num + 2 kv_head_num) * head_size]
    BaseWeight<T> output;  // o_proj [hidden, hidden]
};
