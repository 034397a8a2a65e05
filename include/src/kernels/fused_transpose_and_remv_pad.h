// launchTransposeOutRemovePadding -- same declaration as the reference's
// src/kernels/fused_transpose_and_remv_pad.h:7-10 (declared and tested there, never defined).
// qkv_buf_w_pad [batch, head_num, seq_len, head_size] -> qkv_buf_wo_pad_1 [token_num, head_num, head_size].
#pragma once
#include "src/utils/tensor.h"
template <typename T>
void launchTransposeOutRemovePadding(TensorWrapper<T>* qkv_buf_w_pad, TensorWrapper<int>* padding_offset,
                                     TensorWrapper<T>* qkv_buf_wo_pad_1);
