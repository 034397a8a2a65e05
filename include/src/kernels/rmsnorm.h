// launchRMSNorm -- stand-alone RMSNorm, in place on decoder_out [tokens, hidden].  The reference has
// no separate entry point for it (it is launchFusedAddBiasResidualRMSNorm with a null residual and
// bias, src/kernels/fused_addresidual_norm.cu:51,56,68); this is the same kernel.
#pragma once
#include "src/utils/tensor.h"
#include "src/weights/llama/norm_weights.h"
template <typename T>
void launchRMSNorm(TensorWrapper<T>* decoder_out, LayerNormWeight<T>& norm, float eps);
