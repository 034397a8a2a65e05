// launchCalPaddingoffset -- same declaration as the reference's src/kernels/cal_paddingoffset.h:8-11.
// padding_offset [batch, max_q_len], cum_seqlens [batch + 1], input_lengths [batch].
#pragma once
#include "src/utils/macro.h"
#include "src/utils/tensor.h"
void launchCalPaddingoffset(TensorWrapper<int>* padding_offset, TensorWrapper<int>* cum_seqlens,
                            TensorWrapper<int>* input_lengths);
