// LlamaLayerWeight: device allocation in the reference's shapes, a deterministic dummy fill and the loader of the
// reference's per-tensor .bin files.  Follows src/weights/llama/layer_weights.cc:19-41 (constructor), :45-62 (files)
// and :79-120 (dummy weights) of the reference; HIP runtime underneath.
#include "src/weights/llama/layer_weights.h"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <vector>

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

inline void host_convert(float x, float* p) { *p = x; }
inline void host_convert(float x, half* p) { *p = __float2half(x); }

// `count` fp32 values from `filename` -> T -> device memory at dst   (src/utils/weight_utils.cu:75-140)
template <typename T>
void load_bin(T* dst, size_t count, const std::string& filename) {
    LLM_CHECK_WITH_INFO(dst != nullptr, "no device memory for " + filename);
    std::FILE* f = std::fopen(filename.c_str(), "rb");
    LLM_CHECK_WITH_INFO(f != nullptr, "cannot open weight file " + filename);
    std::vector<float> raw(count);
    const size_t got = std::fread(raw.data(), sizeof(float), count, f);
    std::fclose(f);
    LLM_CHECK_WITH_INFO(got == count, "weight file " + filename + " is shorter than its declared shape");
    std::vector<T> typed(count);
    for (size_t i = 0; i < count; i++) host_convert(raw[i], &typed[i]);
    CHECK(hipMemcpy(dst, typed.data(), count * sizeof(T), hipMemcpyHostToDevice));
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
      bit_size(8 * (int)sizeof(T)),
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
void LlamaLayerWeight<T>::loadWeights(std::string weight_path, WeightType /*weight_type: unused by the reference too*/) {
    const size_t qkv_out = (size_t)(head_num + 2 * kv_head_num) * head_size, h = (size_t)hidden_units;
    load_bin(attn_norm_weight.gamma, h, weight_path + ".input_layernorm.weight.bin");
    load_bin(ffn_norm_weight.gamma, h, weight_path + ".post_attention_layernorm.weight.bin");
    load_bin(self_attn_weight.qkv.data, qkv_out * h, weight_path + ".self_attn.qkv.weight.bin");
    load_bin(self_attn_weight.output.data, h * h, weight_path + ".self_attn.o_proj.weight.bin");
    load_bin(ffn_weight.gateAndup.data, (size_t)2 * inter_size * h, weight_path + ".mlp.gate_up_proj.weight.bin");
    load_bin(ffn_weight.down.data, h * inter_size, weight_path + ".mlp.down_proj.weight.bin");
    if (attn_bias) {
        load_bin(self_attn_weight.qkv.bias, qkv_out, weight_path + ".attention.wqkv.bias.bin");
        load_bin(self_attn_weight.output.bias, h, weight_path + ".attention.wo.bias.bin");
    } else {
        self_attn_weight.qkv.bias = nullptr;
        self_attn_weight.output.bias = nullptr;
        ffn_weight.down.bias = nullptr;
    }
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
