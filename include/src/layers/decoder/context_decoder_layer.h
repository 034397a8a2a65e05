// One LLaMA context-decoder (prefill) layer in C++ over the reference's data model: TensorWrapper /
// TensorMap activations, LlamaLayerWeight weights, a BaseAllocator for the intermediate buffers.
//
// The reference ships the kernels and the weight containers but not the layer code that joins them
// (no src/layers in its tree; its factory constructs an absent Llama<T>, src/utils/model_utils.h:40).
// This class is that join for one layer, in the order the kernels' comments and the weight layout
// imply (src/kernels/linear.cu:7-15, src/weights/llama/layer_weights.cc:19-41,
// src/kernels/fused_addresidual_norm.cu:30,61):
//
//   qkv      = decoder_input x Wqkv^T                      GEMM   [tokens, H] -> [tokens, heads, hs]
//   q, cache = launchAddFusedQKVBiasTransposeRoPEAndConcatKV    bias + RoPE + re-pad + KV append
//   k, v     = launchRepeatKVCache                          cache -> [batch, head_num, max_k_len, hs]
//   scores   = q x k^T (batched GEMM) ; masked, scaled softmax ; ctx = p x v (batched GEMM)
//   packed   = launchTransposeOutRemovePadding              [batch, heads, max_q, hs] -> [tokens, H]
//   attn     = packed x Wo^T                                GEMM
//   launchFusedAddBiasResidualRMSNorm(residual, attn, o-bias, ffn_norm)     residual += attn ; attn := norm
//   gate_up  = attn x Wgate_up^T                            GEMM   -> [tokens, 2, inter]
//   act      = launchAct(gate_up)                           SwiGLU
//   out      = act x Wdown^T                                GEMM
//   launchFusedAddBiasResidualRMSNorm(residual, out, down-bias, next layer's attn_norm)
//
// Every memory-bound step is one of this library's launch* entry points; the four dense GEMMs and the
// two batched attention GEMMs are hipBLASLt calls made here; the softmax between them is a kernel of
// the layers library's own.  That padded, batched attention is the reference's own design
// (src/kernels/linear.cu:67-109, attn_softmax_kernel.cu:50-125) and what fp32 layers and head sizes other
// than 128 and 64 run.  For fp16 heads of 128 or 64 elements the three attention lines (KV broadcast, the two batched
// GEMMs with the softmax, the transpose) are replaced by ONE fused kernel on the matrix cores that reads
// the cache directly and writes the packed rows (launch_fused_context_attention below);
// ISP_LAYERS_ATTENTION=padded in the environment keeps the padded form.
// Everything runs on the null stream, as the reference's launchers do.
//
// forward() tensors (names as the kernels' parameters):
//   inputs   "decoder_input"    T   [num_tokens, hidden]   normalised by this layer's attn_norm; used as scratch
//            "decoder_residual" T   [num_tokens, hidden]   updated in place
//            "padding_offset"   int [batch, max_q_len]     from launchCalPaddingoffset
//            "history_length", "input_length", "context_length"   int [batch]   (device)
//            "layer_id"         int [1]                    host tensor
//   outputs  "decoder_output"   T   [num_tokens, hidden]   the next layer's normalised input
//            "all_k_cache", "all_v_cache"   T [layers, batch, kv_head_num, max_seq_len, head_size]
#pragma once
#include <memory>

#include "src/memory/allocator/base_allocator.h"
#include "src/models/llama/llama_params.h"
#include "src/utils/tensor.h"
#include "src/weights/llama/layer_weights.h"

namespace isp_layers {
class GemmEngine;  // hipBLASLt handle, workspace and per-shape algorithm cache

// The layer's attention softmax, in place on scores [batch, head_num, max_q_len, max_k_len] (device memory,
// null stream): row (b, h, q) becomes softmax(scale * scores) over the keys that query q may see -- key
// positions <= history_length[b] + q and < context_length[b] -- and exactly zero elsewhere; rows of padded
// queries (q >= input_length[b]) become zero.  The mask is computed from the three [batch] length arrays
// instead of being read from a [batch, q, k] tensor (src/kernels/build_casual_mask.cu:5-42,
// attn_softmax_kernel.cu:50-125).  One deliberate departure when a sequence has history: the reference's mask
// also requires k >= context length - query length (build_casual_mask.cu:36), which hides every history key
// (its own comment calls that the mask without multi-turn support and draws the other one); here, and in the
// fused kernel below, a query attends to the history as well.  Identical when history_length = 0.
// Instantiated for float and half.
template <typename T>
void launch_masked_scaled_softmax(T* scores, const int* history_length, const int* input_length,
                                  const int* context_length, int batch, int head_num, int max_q_len,
                                  int max_k_len, float scale);

// The fused causal attention for fp16 heads of hs = 128 or 64 elements (one kernel on the matrix cores in place of KV
// broadcast, q x k^T, the softmax above, p x v and the transpose back to packed tokens; null stream):
//   q_buf            [batch, head_num, max_q_len, hs], rows of padded queries are never read
//   k_cache, v_cache the layer's slice [batch, kv_head_num, max_seq_len, hs] holding history and current keys
//   out              [tokens, head_num, hs], row (first token of b) + q for every q < input_length[b]
// with the same visibility rule as the softmax.  fused_context_attention_supports() says whether a layer
// of these dimensions can use it.
bool fused_context_attention_supports(int head_size, int head_num, int kv_head_num);
void launch_fused_context_attention(const half* q_buf, const half* k_cache, const half* v_cache, half* out,
                                    const int* history_length, const int* input_length, const int* context_length,
                                    int batch, int head_num, int kv_head_num, int head_size, int max_q_len,
                                    int max_k_len, int max_seq_len, int tokens, float scale);
}

template <typename T>
class LlamaContextDecoderLayer {
public:
    LlamaContextDecoderLayer(int head_num, int kv_head_num, int head_size, int inter_size,
                             const LLaMAAttentionStaticParams& attn_params, float rmsnorm_eps,
                             BaseAllocator* allocator);
    ~LlamaContextDecoderLayer();
    LlamaContextDecoderLayer(const LlamaContextDecoderLayer&) = delete;
    LlamaContextDecoderLayer& operator=(const LlamaContextDecoderLayer&) = delete;

    // Makes sure every intermediate buffer holds these extents.  Capacities only grow: a buffer is taken from the
    // allocator again when a call needs more elements than it has, never because the extents merely differ, so
    // after a call at the largest extents forward() allocates nothing (a smaller or differently shaped batch
    // reuses the buffers; the padded positions are re-zeroed with a fill, which is not an allocation).
    void allocForForward(const LLaMAAttentionDynParams& dyn);
    void freeBuf();

    // next_attn_norm: gamma [hidden] of the following layer's attention norm (or the model's final norm).
    void forward(TensorMap& inputs, LlamaLayerWeight<T>& weights, LayerNormWeight<T>& next_attn_norm,
                 TensorMap& outputs, const LLaMAAttentionDynParams& dyn);

    // Device bytes the intermediate buffers of one call with these extents take.
    size_t workspaceBytes(const LLaMAAttentionDynParams& dyn) const;

private:
    int head_num_, kv_head_num_, head_size_, inter_size_, hidden_;
    LLaMAAttentionStaticParams attn_params_;
    float eps_;
    BaseAllocator* allocator_;
    std::unique_ptr<isp_layers::GemmEngine> gemm_;
    bool fused_attention_ = false;  // fp16 heads of 128 or 64: the fused kernel instead of steps 3-5 of the padded form

    LLaMAAttentionDynParams allocated_;   // extents of the last call (what the zeroed padding was laid out for)
    size_t capacity_[9] = {};             // elements each buffer below holds, in their order
    T* qkv_buf_ = nullptr;      // [tokens, head_num + 2 kv_head_num, head_size]
    T* q_buf_ = nullptr;        // [batch, head_num, max_q_len, head_size]
    T* k_all_ = nullptr;        // [batch, head_num, max_k_len, head_size]
    T* v_all_ = nullptr;
    T* scores_ = nullptr;       // [batch, head_num, max_q_len, max_k_len]
    T* ctx_ = nullptr;          // [batch, head_num, max_q_len, head_size]
    T* ctx_packed_ = nullptr;   // [tokens, head_num, head_size]
    T* gate_up_ = nullptr;      // [tokens, 2, inter]
    T* act_ = nullptr;          // [tokens, inter]
};
