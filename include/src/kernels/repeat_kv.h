// launchRepeatKVCache -- same declaration as the reference's src/kernels/repeat_kv.h:7-13.
// k/v_cache_src [num_layers, batch, kv_head_num, max_seq_len, head_size] ->
// k/v_cache_dst [batch, head_num, max_k_len, head_size]; layer_id is a host (CPU) tensor.
#pragma once
#include "src/utils/tensor.h"
template <typename T>
void launchRepeatKVCache(TensorWrapper<T>* k_cache_src, TensorWrapper<T>* v_cache_src,
                         TensorWrapper<int>* context_length, TensorWrapper<int>* layer_id,
                         TensorWrapper<T>* k_cache_dst, TensorWrapper<T>* v_cache_dst);
