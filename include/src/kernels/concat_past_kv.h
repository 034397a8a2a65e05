// launchConcatKVCache -- same declaration as the reference's src/kernels/concat_past_kv.h:7-14.
// k_src, v_src [batch, kv_head_num, max_q_len, head_size]; k_dst, v_dst
// [num_layers, batch, kv_head_num, max_seq_len, head_size]; layer_id is a host (CPU) tensor.
#pragma once
#include "src/utils/tensor.h"
template <typename T>
void launchConcatKVCache(TensorWrapper<T>* k_src, TensorWrapper<T>* v_src, TensorWrapper<int>* layer_id,
                         TensorWrapper<int>* cur_query_length, TensorWrapper<int>* history_length,
                         TensorWrapper<T>* k_dst, TensorWrapper<T>* v_dst);
