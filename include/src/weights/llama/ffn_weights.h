// Feed-forward weights of one LLaMA layer; member names as in the reference's
// src/weights/llama/ffn_weights.h:3-9.  The layer code of this library reads the fused
// `gateAndup` [2 * inter_size, hidden] (rows [0, inter) = gate projection, [inter, 2 inter) = up
// projection, src/weights/llama/layer_weights.cc:33-36) and `down` [hidden, inter_size].
#pragma once
#include "src/weights/base_weights.h"

template <typename T>
struct LLaMAFFNWeights {
    BaseWeight<T> gate;
    BaseWeight<T> up;
    BaseWeight<T> down;
    BaseWeight<T> gateAndup;
};
