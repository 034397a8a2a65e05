// launchFusedAddBiasResidualRMSNorm -- same declaration as the reference's
// src/kernels/fused_addresidual_norm.h:9-15.  In place on `residual` and `decoder_out`
// [tokens, hidden]; bias = norm.bias (may be null), gamma = scale; residual->data may be null
// (plain RMSNorm).  The stored residual includes the bias.
#pragma once
#include "src/utils/tensor.h"
#include "src/utils/vectorize_utils.h"
#include "src/weights/base_weights.h"
#include "src/weights/llama/norm_weights.h"
template <typename T>
void launchFusedAddBiasResidualRMSNorm(TensorWrapper<T>* residual, TensorWrapper<T>* decoder_out,
                                       BaseWeight<T>& norm, T* scale, float eps);
