// Static attention parameters.  The reference includes "src/models/llama/llama_params.h" from
// src/kernels/qkv_bias_and_RoPE.h:5 but ships no such file; the members are the ones its code
// assigns and reads (src/kernels/qkv_bias_and_RoPE.cu:322-325,
// tests/unittests/test_bias_and_RoPE.cu:163-167, src/utils/model_utils.h:25-29).
#pragma once
struct LLaMAAttentionStaticParams {
    int rotary_embedding_dim = 128;
    float rotary_embedding_base = 10000.0f;
    int max_position_embeddings = 2048;
    bool use_dynamic_ntk = false;  // placeholder in the reference as well
};

// Per-call extents of the attention / decoder layers.  The reference's kernels take them from tensor
// shapes; the layer code (which the reference does not ship) needs them before the tensors exist,
// to size its buffers.
struct LLaMAAttentionDynParams {
    int batch_size = 0;
    int num_tokens = 0;   // valid (un-padded) tokens of the batch
    int max_q_len = 0;    // longest query of the batch: the padded sequence extent of q
    int max_k_len = 0;    // longest context (history + query) of the batch
    int num_layers = 0;
    bool is_ctx = true;
};
