// LlamaContextDecoder: the loop over LlamaContextDecoderLayer (see the header for the sequence).
#include "src/layers/decoder/context_decoder.h"

#include <string>

#include "src/kernels/cal_paddingoffset.h"
#include "src/kernels/rmsnorm.h"
#include "src/utils/macro.h"

template <typename T>
LlamaContextDecoder<T>::LlamaContextDecoder(int head_num, int kv_head_num, int head_size, int inter_size,
                                            int num_layers, const LLaMAAttentionStaticParams& attn_params,
                                            float rmsnorm_eps, BaseAllocator* allocator)
    : num_layers_(num_layers), hidden_(head_num * head_size), eps_(rmsnorm_eps), allocator_(allocator),
      layer_(new LlamaContextDecoderLayer<T>(head_num, kv_head_num, head_size, inter_size, attn_params, rmsnorm_eps,
                                             allocator)) {
    LLM_CHECK_WITH_INFO(num_layers > 0, "a decoder needs at least one layer");
    LLM_CHECK_WITH_INFO(allocator != nullptr, "a decoder needs an allocator for its buffers");
}

template <typename T>
LlamaContextDecoder<T>::~LlamaContextDecoder() {
    freeBuf();
}

template <typename T>
void LlamaContextDecoder<T>::allocForForward(const LLaMAAttentionDynParams& d) {
    freeBuf();
    const size_t rows = (size_t)d.num_tokens * hidden_;
    padding_offset_ = static_cast<int*>(allocator_->UnifyMalloc(nullptr, sizeof(int) * d.batch_size * d.max_q_len, false));
    cum_seqlens_ = static_cast<int*>(allocator_->UnifyMalloc(nullptr, sizeof(int) * (d.batch_size + 1), false));
    residual_ = static_cast<T*>(allocator_->UnifyMalloc(nullptr, sizeof(T) * rows, false));
    hidden_a_ = static_cast<T*>(allocator_->UnifyMalloc(nullptr, sizeof(T) * rows, false));
    hidden_b_ = static_cast<T*>(allocator_->UnifyMalloc(nullptr, sizeof(T) * rows, false));
    allocated_ = d;
}

template <typename T>
void LlamaContextDecoder<T>::freeBuf() {
    void* all[] = {padding_offset_, cum_seqlens_, residual_, hidden_a_, hidden_b_};
    for (void* p : all)
        if (p) allocator_->UnifyFree(p, false);
    padding_offset_ = cum_seqlens_ = nullptr;
    residual_ = hidden_a_ = hidden_b_ = nullptr;
    allocated_ = LLaMAAttentionDynParams();
}

template <typename T>
void LlamaContextDecoder<T>::forward(TensorMap& inputs, const std::vector<LlamaLayerWeight<T>*>& layer_weights,
                                     LayerNormWeight<T>& final_norm, TensorMap& outputs,
                                     const LLaMAAttentionDynParams& dyn) {
    for (const char* name : {"decoder_input", "history_length", "input_length", "context_length"})
        LLM_CHECK_WITH_INFO(inputs.isExist(name), std::string("missing input tensor: ") + name);
    for (const char* name : {"decoder_output", "all_k_cache", "all_v_cache"})
        LLM_CHECK_WITH_INFO(outputs.isExist(name), std::string("missing output tensor: ") + name);
    LLM_CHECK_WITH_INFO((int)layer_weights.size() == num_layers_, "one LlamaLayerWeight per layer is required");
    for (auto* w : layer_weights) LLM_CHECK_WITH_INFO(w != nullptr, "a layer's weights are missing");
    Tensor* in_any = inputs.at("decoder_input");
    Tensor* out_any = outputs.at("decoder_output");
    LLM_CHECK_WITH_INFO(in_any->dtype == getTensorType<T>() && out_any->dtype == getTensorType<T>(),
                        "decoder_input / decoder_output have the wrong element type");
    auto* decoder_input = static_cast<TensorWrapper<T>*>(in_any);
    auto* decoder_output = static_cast<TensorWrapper<T>*>(out_any);
    const int tokens = dyn.num_tokens, batch = dyn.batch_size;
    LLM_CHECK_WITH_INFO(decoder_input->shape.size() == 2 && decoder_input->shape[0] == tokens &&
                            decoder_input->shape[1] == hidden_ && decoder_output->shape == decoder_input->shape,
                        "decoder_input / decoder_output should be [num_tokens, hidden]");
    LLM_CHECK_WITH_INFO(inputs.at("input_length")->dtype == getTensorType<int>() &&
                            inputs.at("input_length")->shape.size() == 1 && inputs.at("input_length")->shape[0] == batch,
                        "input_length should be int [batch]");
    Tensor* k_cache = outputs.at("all_k_cache");
    LLM_CHECK_WITH_INFO(k_cache->shape.size() == 5 && k_cache->shape[0] >= num_layers_,
                        "the KV cache should be [layers, batch, kv_head_num, max_seq_len, head_size] with a slice per layer");
    if (tokens == 0) return;
    if (dyn.num_tokens > allocated_.num_tokens || dyn.batch_size > allocated_.batch_size ||
        dyn.max_q_len != allocated_.max_q_len)
        allocForForward(dyn);

    const DataType dt = getTensorType<T>();
    const size_t row_bytes = sizeof(T) * (size_t)tokens * hidden_;
    auto* input_length = static_cast<TensorWrapper<int>*>(inputs.at("input_length"));
    TensorWrapper<int> padding_offset(Device::GPU, getTensorType<int>(), {batch, dyn.max_q_len}, padding_offset_);
    TensorWrapper<int> cum_seqlens(Device::GPU, getTensorType<int>(), {batch + 1}, cum_seqlens_);
    launchCalPaddingoffset(&padding_offset, &cum_seqlens, input_length);

    // residual = the embedded tokens; x = their RMSNorm by the first layer's attention norm
    CHECK(hipMemcpyAsync(residual_, decoder_input->data, row_bytes, hipMemcpyDeviceToDevice, nullptr));
    CHECK(hipMemcpyAsync(hidden_a_, decoder_input->data, row_bytes, hipMemcpyDeviceToDevice, nullptr));
    TensorWrapper<T> first(Device::GPU, dt, {tokens, hidden_}, hidden_a_);
    LLM_CHECK_WITH_INFO(layer_weights[0]->attn_norm_weight.gamma != nullptr, "norm weights are not loaded");
    launchRMSNorm(&first, layer_weights[0]->attn_norm_weight, eps_);

    TensorWrapper<T> residual(Device::GPU, dt, {tokens, hidden_}, residual_);
    T* from = hidden_a_;
    T* to = hidden_b_;
    for (int l = 0; l < num_layers_; l++) {
        const bool last = l + 1 == num_layers_;
        TensorWrapper<T> x(Device::GPU, dt, {tokens, hidden_}, from);
        TensorWrapper<T> y(Device::GPU, dt, {tokens, hidden_}, last ? decoder_output->data : to);
        int layer_value = l;
        TensorWrapper<int> layer_id(Device::CPU, getTensorType<int>(), {1}, &layer_value);
        TensorMap layer_inputs{{"decoder_input", &x},
                               {"decoder_residual", &residual},
                               {"padding_offset", &padding_offset},
                               {"history_length", inputs.at("history_length")},
                               {"input_length", inputs.at("input_length")},
                               {"context_length", inputs.at("context_length")},
                               {"layer_id", &layer_id}};
        TensorMap layer_outputs{{"decoder_output", &y},
                                {"all_k_cache", outputs.at("all_k_cache")},
                                {"all_v_cache", outputs.at("all_v_cache")}};
        layer_->forward(layer_inputs, *layer_weights[l], last ? final_norm : layer_weights[l + 1]->attn_norm_weight,
                        layer_outputs, dyn);
        T* t = from;
        from = to;
        to = t;
    }
}

template class LlamaContextDecoder<float>;
template class LlamaContextDecoder<half>;
