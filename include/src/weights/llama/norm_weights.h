// RMSNorm scale vector of one normalisation point (attention norm, FFN norm or the final norm).
// Same type and member name as the reference's src/weights/llama/norm_weights.h; `gamma` points to
// `hidden` elements on the device and defaults to nullptr here (the reference leaves it unset).
// launchRMSNorm takes this struct; launchFusedAddBiasResidualRMSNorm takes the raw pointer as its
// `scale` argument, as in the reference.
#pragma once

template <typename T>
struct LayerNormWeight {
    T* gamma = nullptr;
};
