// launchAct -- same declaration as the reference's src/kernels/act_kernel.h:8-9 (SwiGLU).
// input [tokens, 2, inter] -> out [tokens, inter]; throws unless input->shape[1] == 2.
#pragma once
#include "src/utils/tensor.h"
#include "src/utils/vectorize_utils.h"
template <typename T>
void launchAct(TensorWrapper<T>* input, TensorWrapper<T>* out);
