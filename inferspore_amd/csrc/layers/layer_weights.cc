// LlamaLayerWeight: device allocation in the reference's shapes and a deterministic dummy fill.
// Follows src/weights/llama/layer_weights.cc:19-41 (constructor) and :79-120 (dummy weights) of the
// reference; HIP runtime underneath.
#include "src/weights/llama/layer_weights.h"

#include <algorithm>
#include <cmath>
#include <cstdint>

#include "src/utils/macro.h"

namespace {

template <typename T>
T* device_array(size_t n) {
    T* p = nullptr;
    CHECK(hipMalloc(reinterpret_cast<void**>(&p), n * sizeof(T)));
    return p;
}

__device__ inline void to_storage(float x, float* p) { *p = x; }
__device__ inline void to_storage(float x, half* p) { *p = __float2half(x); }

// value i of stream `tag`: a fixed integer hash mapped to [-scale, scale) (+ shift); filled on the device
// (a 7B-shaped layer holds 200 M weights)
template <typename T>
__global__ void fill_kernel(T* dst, size_t n, uint32_t tag, float scale, float shift) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        uint32_t x = (uint32_t)i * 2654435761u + tag * 40503u + 12345u;
        x ^= x >> 15;
        x *= 2246822519u;
        x ^= x >> 13;
        const float u = (float)(x >> 8) * (1.0f / 16777216.0f) - 0.5f;  // [-0.5, 0.5)
        to_storage(shift + 2.0f * scale * u, dst + i);
    }
}

template <typename T>
void fill(T* dst, size_t n, uint32_t tag, float scale, float shift) {
    if (n == 0) return;
    const unsigned blocks = (unsigned)std::min<size_t>((n + 255) / 256, 65536);
    hipLaunchKernelGGL(fill_kernel<T>, dim3(blocks), dim3(256), 0, nullptr, dst, n, tag, scale, shift);
    CHECK(hipGetLastError());
}

}  // namespace

template <typename T>
LlamaLayerWeight<T>::LlamaLayerWeight(int head_num, int kv_head_num, int head_size, int inter_size,
                                      WeightType weight_type, bool attn_bias)
    : head_num(head_num),
      kv_head_num(kv_head_num),
      head_size(head_size),
      hidden_units(head_num * head_size),
      inter_size(inter_size),
      weight_type(weight_type),
      attn_bias(attn_bias) {
    const int qkv_out = (head_num + 2 * kv_head_num) * head_size;
    attn_norm_weight.gamma = device_array<T>(hidden_units);
    ffn_norm_weight.gamma = device_array<T>(hidden_units);
    self_attn_weight.qkv.type = weight_type;
    self_attn_weight.qkv.shape = {qkv_out, hidden_units};
    self_attn_weight.qkv.data = device_array<T>((size_t)qkv_out * hidden_units);
    self_attn_weight.output.type = weight_type;
    self_attn_weight.output.shape = {hidden_units, hidden_units};
    self_attn_weight.output.data = device_array<T>((size_t)hidden_units * hidden_units);
    if (attn_bias) {
        self_attn_weight.qkv.bias = device_array<T>(qkv_out);
        self_attn_weight.output.bias = device_array<T>(hidden_units);
    }
    ffn_weight.gateAndup.type = weight_type;
    ffn_weight.gateAndup.shape = {2 * inter_size, hidden_units};
    ffn_weight.gateAndup.data = device_array<T>((size_t)2 * inter_size * hidden_units);
    ffn_weight.down.type = weight_type;
    ffn_weight.down.shape = {hidden_units, inter_size};
    ffn_weight.down.data = device_array<T>((size_t)hidden_units * inter_size);
}

template <typename T>
LlamaLayerWeight<T>::~LlamaLayerWeight() {
    T* all[] = {attn_norm_weight.gamma,        ffn_norm_weight.gamma,      self_attn_weight.qkv.data,
                self_attn_weight.qkv.bias,     self_attn_weight.output.data, self_attn_weight.output.bias,
                ffn_weight.gateAndup.data,     ffn_weight.down.data};
    for (T* p : all)
        if (p) (void)hipFree(p);
}

template <typename T>
void LlamaLayerWeight<T>::loadWeights() {
    const int qkv_out = (head_num + 2 * kv_head_num) * head_size;
    const float wh = 1.0f / std::sqrt((float)hidden_units), wi = 1.0f / std::sqrt((float)inter_size);
    fill(attn_norm_weight.gamma, (size_t)hidden_units, 1, 0.5f, 1.0f);
    fill(ffn_norm_weight.gamma, (size_t)hidden_units, 2, 0.5f, 1.0f);
    fill(self_attn_weight.qkv.data, (size_t)qkv_out * hidden_units, 3, 1.7f * wh, 0.0f);
    fill(self_attn_weight.output.data, (size_t)hidden_units * hidden_units, 4, 1.7f * wh, 0.0f);
    fill(ffn_weight.gateAndup.data, (size_t)2 * inter_size * hidden_units, 5, 1.7f * wh, 0.0f);
    fill(ffn_weight.down.data, (size_t)hidden_units * inter_size, 6, 1.7f * wi, 0.0f);
    if (attn_bias) {
        fill(self_attn_weight.qkv.bias, (size_t)qkv_out, 7, 0.02f, 0.0f);
        fill(self_attn_weight.output.bias, (size_t)hidden_units, 8, 0.02f, 0.0f);
    }
    CHECK(hipDeviceSynchronize());
}

template class LlamaLayerWeight<float>;
template class LlamaLayerWeight<half>;
