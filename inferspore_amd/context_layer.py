"""Caller-side glue: one LLaMA context-decoder (prefill) layer built from this library's kernels.

The reference ships the kernels but not the layer code that calls them (its `src/layers` and
`Llama<T>` class are absent); this module is the call sequence its kernel comments and weight layout
imply (fused QKV weight `[H, 3H]`, fused gate/up weight `[H, 2I]`, reference
src/weights/llama/layer_weights.cc:19-62), so that the kernels can be exercised and timed in the
order a model runs them:

    normed, residual                       (packed [tokens, H]; `normed` = RMSNorm(residual) by attn_norm)
    qkv      = normed @ Wqkv                                 library GEMM (out of this library's scope)
    q, cache += k, v = add_fused_qkv_bias_transpose_rope_and_append(qkv)    * this library
    k_all, v_all = repeat(cache)                             * this library
    ctx      = softmax(q k^T / sqrt(d) + mask) v             library attention (out of scope)
    packed   = transpose_out_remove_padding(ctx)             * this library
    attn_out = packed @ Wo                                   library GEMM
    residual, normed2 = fused_add_bias_residual_rmsnorm(residual, attn_out, ffn_norm)      * this library
    act      = SwiGLU(normed2 @ Wgate_up)                    library GEMM + * this library
    ffn_out  = act @ Wdown                                   library GEMM
    residual, normed_next = fused_add_bias_residual_rmsnorm(residual, ffn_out, next attn_norm)   * this library

Dense contractions and attention are deliberately left to torch's library calls (hipBLASLt GEMMs,
scaled_dot_product_attention); everything marked * goes through the C ABI.  All work is issued on
torch's current stream.
"""
import math

import torch

from . import ops


class LayerWeights:
    """Weights of one layer in the reference's fused layout."""

    def __init__(self, hidden, inter, dtype, device="cuda", generator=None, qkv_bias=False):
        def w(*shape, scale):
            return (scale * torch.randn(shape, device=device, generator=generator)).to(dtype)

        self.qkv = w(hidden, 3 * hidden, scale=hidden ** -0.5)
        self.qkv_bias = w(3 * hidden, scale=0.02) if qkv_bias else None
        self.o = w(hidden, hidden, scale=hidden ** -0.5)
        self.gate_up = w(hidden, 2 * inter, scale=hidden ** -0.5)   # columns [0, I) gate, [I, 2I) up
        self.down = w(inter, hidden, scale=inter ** -0.5)
        self.attn_norm = (0.5 + torch.rand(hidden, device=device, generator=generator)).to(dtype)
        self.ffn_norm = (0.5 + torch.rand(hidden, device=device, generator=generator)).to(dtype)


class BatchState:
    """Padding bookkeeping of one ragged prefill batch plus the buffers a layer needs."""

    def __init__(self, lengths, max_q_len, head_num, kv_head_num, head_size, inter, max_seq_len, layers, dtype,
                 history=None):
        dev = "cuda"
        self.batch = len(lengths)
        self.max_q_len, self.max_seq_len = max_q_len, max_seq_len
        self.head_num, self.kv_head_num, self.head_size = head_num, kv_head_num, head_size
        self.lengths = torch.as_tensor(lengths, dtype=torch.int32).to(dev)
        self.history = (torch.zeros(self.batch, dtype=torch.int32, device=dev) if history is None
                        else torch.as_tensor(history, dtype=torch.int32).to(dev))
        self.context = self.lengths + self.history
        self.tokens = int(sum(lengths))
        self.max_k_len = int(max(int(l) + int(h) for l, h in zip(lengths, self.history.tolist())))
        self.padding_offset = torch.zeros((self.batch, max_q_len), dtype=torch.int32, device=dev)
        self.cum_seqlens = torch.zeros(self.batch + 1, dtype=torch.int32, device=dev)
        ops.cal_padding_offset(self.padding_offset, self.cum_seqlens, self.lengths)
        hidden = head_num * head_size
        z = lambda *s: torch.zeros(s, dtype=dtype, device=dev)
        self.q = z(self.batch, head_num, max_q_len, head_size)
        self.k_cache = z(layers, self.batch, kv_head_num, max_seq_len, head_size)
        self.v_cache = z(layers, self.batch, kv_head_num, max_seq_len, head_size)
        self.k_all = z(self.batch, head_num, self.max_k_len, head_size)
        self.v_all = z(self.batch, head_num, self.max_k_len, head_size)
        self.packed_ctx = z(self.tokens, head_num, head_size)
        self.act = z(self.tokens, inter)
        # additive attention mask [batch, 1, max_q_len, max_k_len]: query s of sequence b sees keys
        # 0 .. history[b] + s, and only when s is a valid position
        s = torch.arange(max_q_len, device=dev)[None, :, None]
        kpos = torch.arange(self.max_k_len, device=dev)[None, None, :]
        hist = self.history[:, None, None]
        visible = (kpos <= hist + s) & (s < self.lengths[:, None, None])
        self.mask = torch.zeros((self.batch, 1, max_q_len, self.max_k_len), dtype=dtype, device=dev)
        self.mask.masked_fill_(~visible[:, None], float("-inf"))
        # fully padded query rows would be all -inf: let them see key 0 (their output is discarded)
        self.mask[:, :, :, 0].masked_fill_(~(s[:, :, 0] < self.lengths[:, None])[:, None], 0.0)
        del hidden


def context_decoder_layer(normed, residual, w, state, layer_id, next_norm_gamma, rotary_dim=128,
                          rotary_base=10000.0, eps=1e-5):
    """Runs one prefill layer.  `normed` and `residual` are packed [tokens, H]; `residual` is updated in
    place; returns the next layer's normalised input (a new tensor)."""
    st = state
    qkv = normed @ w.qkv                                                       # [tokens, 3H]
    qkv = qkv.view(st.tokens, st.head_num + 2 * st.kv_head_num, st.head_size)
    # bias + RoPE + re-pad of q, with k and v written straight into the cache (one launch, no padded k / v)
    ops.add_fused_qkv_bias_transpose_rope_and_append(st.q, None, None, st.k_cache, st.v_cache, layer_id, qkv,
                                                     w.qkv_bias, st.padding_offset, st.history, st.lengths,
                                                     rotary_dim, rotary_base)
    ops.repeat_kv_cache(st.k_cache, st.v_cache, st.context, layer_id, st.k_all, st.v_all)
    ctx = torch.nn.functional.scaled_dot_product_attention(st.q, st.k_all, st.v_all, attn_mask=st.mask,
                                                           scale=1.0 / math.sqrt(st.head_size))
    ops.transpose_out_remove_padding(ctx.contiguous(), st.padding_offset, st.packed_ctx)
    attn_out = st.packed_ctx.view(st.tokens, -1) @ w.o
    ops.fused_add_bias_residual_rmsnorm(residual, attn_out, None, w.ffn_norm, eps)   # attn_out := normed
    gate_up = (attn_out @ w.gate_up).view(st.tokens, 2, -1)
    ops.act(gate_up, st.act)
    ffn_out = st.act @ w.down
    ops.fused_add_bias_residual_rmsnorm(residual, ffn_out, None, next_norm_gamma, eps)
    return ffn_out
