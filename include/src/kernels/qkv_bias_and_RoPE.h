// launchAddFusedQKVBiasTransposeAndRoPE -- same declaration as the reference's
// src/kernels/qkv_bias_and_RoPE.h:10-20.  Shapes are taken from the tensors as the reference's
// launcher does (src/kernels/qkv_bias_and_RoPE.cu:298-304):
//   QKV [token_num, head_num + 2 kv_head_num, head_size];  q_buf [batch, head_num, seq_len, head_size];
//   k_buf, v_buf [batch, kv_head_num, seq_len, head_size];  bias = qkv.bias (may be null).
#pragma once
#include "src/models/llama/llama_params.h"
#include "src/utils/tensor.h"
#include "src/utils/vectorize_utils.h"
#include "src/weights/base_weights.h"
template <typename T>
void launchAddFusedQKVBiasTransposeAndRoPE(TensorWrapper<T>* q_buf, TensorWrapper<T>* k_buf,
                                           TensorWrapper<T>* v_buf, TensorWrapper<T>* QKV,
                                           BaseWeight<T>& qkv, TensorWrapper<int>* padding_offset,
                                           TensorWrapper<int>* history_length,
                                           TensorWrapper<int>* input_length,
                                           LLaMAAttentionStaticParams& params);

// The same step with launchConcatKVCache fused in (no counterpart in the reference, which runs the two
// launchers one after the other, src/kernels/concat_past_kv.cu:76-113): the k and v rows go straight
// to k_cache / v_cache [layers, batch, kv_head_num, max_seq_len, head_size] at layer layer_id (a host
// tensor, as in launchConcatKVCache) and row history_length[b] + s; no padded k / v buffers are
// written.  kv_head_num and max_seq_len are taken from the cache's shape.
template <typename T>
void launchAddFusedQKVBiasTransposeRoPEAndConcatKV(TensorWrapper<T>* q_buf, TensorWrapper<T>* QKV,
                                                   BaseWeight<T>& qkv,
                                                   TensorWrapper<int>* padding_offset,
                                                   TensorWrapper<int>* history_length,
                                                   TensorWrapper<int>* input_length,
                                                   TensorWrapper<int>* layer_id,
                                                   TensorWrapper<T>* k_cache,
                                                   TensorWrapper<T>* v_cache,
                                                   LLaMAAttentionStaticParams& params);

// launchRoPE -- same declaration as the reference's src/kernels/qkv_bias_and_RoPE.h:22-25 (decode
// phase): in-place rotate-half RoPE on qkv_buf [1, 96, 128] at timestep step - 1; `step` is a host
// (CPU) tensor.  The reference's checks (batch 1, 96 heads of 128, 32 q heads) are kept.
template <typename T>
void launchRoPE(TensorWrapper<T>* qkv_buf, TensorWrapper<int>* step,
                LLaMAAttentionStaticParams& static_params);
