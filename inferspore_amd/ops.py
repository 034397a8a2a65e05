"""The C ABI called on torch tensors (device memory and the current stream come from torch).

Names and argument meaning mirror the reference's `launch*` functions; shapes are derived from the
tensors exactly as the reference's launchers derive them from `TensorWrapper::shape`.  All calls are
asynchronous on torch's current stream.  Nothing here computes on the host.

Every wrapper checks dtypes and operand extents on the host before it launches: the kernels trust
their arguments, so a mis-shaped tensor has to become a Python exception here, not an out-of-bounds
access on the device.  (The reference's launchers check less; see each function.)
"""
import torch

from . import capi

_SUFFIX = {torch.float16: "f16", torch.float32: "f32"}


def _suffix(t):
    try:
        return _SUFFIX[t.dtype]
    except KeyError:
        raise TypeError("inferspore_amd kernels take float16 or float32 tensors, got %s" % t.dtype)


def _expect(ok, what):
    if not ok:
        raise RuntimeError("inferspore_amd: " + what)


def _dev(*tensors):
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("inferspore_amd: tensors must live on the GPU (no CPU path exists)")
        if not t.is_contiguous():
            raise RuntimeError("inferspore_amd: tensors must be contiguous")


def _p(t):
    return None if t is None else t.data_ptr()


def _same_dtype(ref, *tensors):
    for t in tensors:
        if t is not None and t.dtype != ref.dtype:
            raise TypeError("inferspore_amd: operand dtype %s does not match %s" % (t.dtype, ref.dtype))


def _int32(*tensors):
    for t in tensors:
        if t is not None and t.dtype != torch.int32:
            raise TypeError("inferspore_amd: index / length tensors must be int32, got %s" % t.dtype)


def _stream():
    return torch.cuda.current_stream().cuda_stream


def input_embedding(input_ids, output, embed_table, check_bounds=True):
    """launchInputEmbedding: output[t, :] = embed_table[input_ids[t], :]."""
    _int32(input_ids)
    _suffix(output)
    _expect(output.dim() == 2 and embed_table.dim() == 2 and input_ids.dim() == 1,
            "input_embedding takes ids [tokens], output [tokens, hidden], table [vocab, hidden]")
    if output.shape[0] != input_ids.shape[0]:
        raise RuntimeError("input ids 1st shape should equal to 1st shape of output")   # input_embedding.cu:35
    if output.dtype != embed_table.dtype:
        raise TypeError("output and table dtypes differ")
    _expect(embed_table.shape[1] == output.shape[1], "table rows and output rows differ in length")
    _dev(input_ids, output, embed_table)
    fn = getattr(capi.lib(), "isp_embedding_" + _suffix(output))
    vocab = embed_table.shape[0] if check_bounds else 0
    capi.check(fn(_p(input_ids), _p(output), _p(embed_table), output.shape[0], output.shape[1],
                  vocab, _stream()), "isp_embedding")
    return output


def cal_padding_offset(padding_offset, cum_seqlens, input_lengths):
    """launchCalPaddingoffset: padding_offset [batch, max_q_len], cum_seqlens [batch + 1]."""
    _expect(padding_offset.dim() == 2 and cum_seqlens.dim() == 1 and input_lengths.dim() == 1,
            "cal_padding_offset takes padding_offset [batch, max_q_len], cum_seqlens [batch + 1], lengths [batch]")
    batch, max_q_len = padding_offset.shape
    if batch != input_lengths.shape[0]:
        raise RuntimeError("input lenghts numbers should equal to padding offset bs dim!")   # cal_paddingoffset.cu:55
    if batch != cum_seqlens.shape[0] - 1:
        raise RuntimeError("cum seqlen numbers should equal to padding offset bs dim + 1!")  # cal_paddingoffset.cu:56
    for t in (padding_offset, cum_seqlens, input_lengths):
        if t.dtype != torch.int32:
            raise TypeError("padding-offset tensors must be int32")
    _dev(padding_offset, cum_seqlens, input_lengths)
    capi.check(capi.lib().isp_cal_padding_offset(_p(padding_offset), _p(cum_seqlens),
                                                 _p(input_lengths), batch, max_q_len, _stream()),
               "isp_cal_padding_offset")
    return padding_offset, cum_seqlens


def rmsnorm(x, gamma, eps):
    """In-place RMSNorm of x [tokens, hidden]."""
    _same_dtype(x, gamma)
    _expect(x.dim() == 2, "rmsnorm takes x [tokens, hidden]")
    _expect(gamma.numel() == x.shape[1], "gamma must hold one value per hidden column")
    _dev(x, gamma)
    fn = getattr(capi.lib(), "isp_rmsnorm_" + _suffix(x))
    capi.check(fn(_p(x), _p(gamma), float(eps), x.shape[0], x.shape[1], _stream()), "isp_rmsnorm")
    return x


def fused_add_bias_residual_rmsnorm(residual, decoder_out, bias, gamma, eps, flags=0):
    """launchFusedAddBiasResidualRMSNorm: in place on residual (may be None) and decoder_out."""
    _same_dtype(decoder_out, residual, bias, gamma)
    _expect(decoder_out.dim() == 2, "fused norm takes decoder_out [tokens, hidden]")
    hidden = decoder_out.shape[1]
    _expect(residual is None or tuple(residual.shape) == tuple(decoder_out.shape),
            "residual and decoder_out must have the same shape")
    _expect(gamma.numel() == hidden, "gamma must hold one value per hidden column")
    _expect(bias is None or bias.numel() == hidden, "bias must hold one value per hidden column")
    _expect(residual is None or residual.data_ptr() != decoder_out.data_ptr(),
            "residual and decoder_out must be distinct buffers")
    _dev(residual, decoder_out, bias, gamma)
    fn = getattr(capi.lib(), "isp_fused_add_bias_residual_rmsnorm_" + _suffix(decoder_out))
    capi.check(fn(_p(residual), _p(decoder_out), _p(bias), _p(gamma), float(eps),
                  decoder_out.shape[0], hidden, int(flags), _stream()),
               "isp_fused_add_bias_residual_rmsnorm")
    return residual, decoder_out


def _qkv_shapes(q_buf, k_buf, v_buf, qkv, qkv_bias, padding_offset, history_length, input_length, kv_optional):
    _expect(qkv.dim() == 3 and q_buf.dim() == 4, "qkv must be [tokens, heads, head_size], q_buf [batch, heads, seq, head_size]")
    token_num, qkv_head_num, head_size = qkv.shape
    batch, head_num, seq_len = q_buf.shape[0], q_buf.shape[1], q_buf.shape[2]
    _expect(qkv_head_num >= head_num and (qkv_head_num - head_num) % 2 == 0,
            "packed head count must be head_num + 2 * kv_head_num")
    kv_head_num = (qkv_head_num - head_num) // 2
    _expect(q_buf.shape[3] == head_size, "q_buf head size differs from qkv's")
    for name, t in (("k_buf", k_buf), ("v_buf", v_buf)):
        if t is None:
            _expect(kv_optional, name + " is required")
        else:
            _expect(tuple(t.shape) == (batch, kv_head_num, seq_len, head_size),
                    name + " must be [batch, kv_head_num, seq_len, head_size]")
    _expect((k_buf is None) == (v_buf is None), "k_buf and v_buf must both be given or both be None")
    _expect(qkv_bias is None or qkv_bias.numel() == qkv_head_num * head_size,
            "qkv_bias must hold one value per packed column")
    _expect(padding_offset.numel() >= token_num, "padding_offset is shorter than the token count")
    _expect(history_length.numel() >= batch, "history_length is shorter than the batch")
    _expect(input_length is None or input_length.numel() >= batch, "input_length is shorter than the batch")
    return token_num, head_size, batch, head_num, seq_len, kv_head_num


def add_fused_qkv_bias_transpose_and_rope(q_buf, k_buf, v_buf, qkv, qkv_bias, padding_offset,
                                          history_length, input_length, rotary_embedding_dim,
                                          rotary_embedding_base, max_position_embeddings=2048,
                                          use_dynamic_ntk=False):
    """launchAddFusedQKVBiasTransposeAndRoPE; shapes as the reference derives them
    (qkv_bias_and_RoPE.cu:298-304)."""
    _same_dtype(qkv, q_buf, k_buf, v_buf, qkv_bias)
    _int32(padding_offset, history_length, input_length)
    token_num, head_size, batch, head_num, seq_len, kv_head_num = _qkv_shapes(
        q_buf, k_buf, v_buf, qkv, qkv_bias, padding_offset, history_length, input_length, kv_optional=False)
    _dev(q_buf, k_buf, v_buf, qkv, qkv_bias, padding_offset, history_length, input_length)
    fn = getattr(capi.lib(), "isp_qkv_bias_rope_transpose_" + _suffix(qkv))
    capi.check(fn(_p(q_buf), _p(k_buf), _p(v_buf), _p(qkv), _p(qkv_bias), _p(padding_offset),
                  _p(history_length), _p(input_length), batch, seq_len, token_num, head_num,
                  kv_head_num, head_size, int(rotary_embedding_dim), float(rotary_embedding_base),
                  int(max_position_embeddings), int(bool(use_dynamic_ntk)), _stream()),
               "isp_qkv_bias_rope_transpose")
    return q_buf, k_buf, v_buf


def add_fused_qkv_bias_transpose_rope_and_append(q_buf, k_buf, v_buf, k_cache, v_cache, layer_id, qkv, qkv_bias,
                                                 padding_offset, history_length, input_length,
                                                 rotary_embedding_dim, rotary_embedding_base):
    """launchAddFusedQKVBiasTransposeAndRoPE with launchConcatKVCache fused in: k_buf / v_buf may both be
    None (the k and v rows then go to the cache only).
    k_cache, v_cache [layers, batch, kv_head_num, max_seq_len, head_size]."""
    _same_dtype(qkv, q_buf, k_buf, v_buf, k_cache, v_cache, qkv_bias)
    _int32(padding_offset, history_length, input_length)
    _expect(input_length is not None, "input_length is required")
    token_num, head_size, batch, head_num, seq_len, kv_head_num = _qkv_shapes(
        q_buf, k_buf, v_buf, qkv, qkv_bias, padding_offset, history_length, input_length, kv_optional=True)
    _expect(k_cache.dim() == 5 and tuple(k_cache.shape) == tuple(v_cache.shape) and
            tuple(k_cache.shape[1:3]) == (batch, kv_head_num) and k_cache.shape[4] == head_size,
            "caches must be [layers, batch, kv_head_num, max_seq_len, head_size]")
    _expect(0 <= int(layer_id) < k_cache.shape[0], "layer_id outside the cache")
    _dev(q_buf, k_buf, v_buf, k_cache, v_cache, qkv, qkv_bias, padding_offset, history_length, input_length)
    fn = getattr(capi.lib(), "isp_qkv_bias_rope_transpose_append_" + _suffix(qkv))
    capi.check(fn(_p(q_buf), _p(k_buf), _p(v_buf), _p(k_cache), _p(v_cache), int(layer_id), k_cache.shape[3], _p(qkv),
                  _p(qkv_bias), _p(padding_offset), _p(history_length), _p(input_length), batch, seq_len, token_num,
                  head_num, kv_head_num, head_size, int(rotary_embedding_dim), float(rotary_embedding_base), _stream()),
               "isp_qkv_bias_rope_transpose_append")
    return q_buf, k_cache, v_cache


def act(input, out):
    """launchAct (SwiGLU): input [tokens, 2, inter] -> out [tokens, inter]."""
    _same_dtype(input, out)
    _expect(input.dim() == 3, "SwiGLU input must have shape [tokens, 2, inter]")
    if input.shape[1] != 2:
        raise RuntimeError("SwiGLU input must have shape [tokens, 2, inter]")   # act_kernel.cu:61
    _expect(tuple(out.shape) == (input.shape[0], input.shape[2]), "SwiGLU output must be [tokens, inter]")
    _dev(input, out)
    fn = getattr(capi.lib(), "isp_swiglu_" + _suffix(input))
    capi.check(fn(_p(input), _p(out), input.shape[0], input.shape[2], _stream()), "isp_swiglu")
    return out


def rope(qkv_buf, step, head_num, rotary_embedding_dim, rotary_embedding_base):
    """launchRoPE (decode): in place on qkv_buf [batch, head_num + 2 kv_head_num, head_size]; `step` is a
    host integer (the reference reads it from a CPU tensor)."""
    _expect(qkv_buf.dim() == 3, "qkv_buf must be [batch, heads, head_size]")
    batch, qkv_head_num, head_size = qkv_buf.shape
    _expect(qkv_head_num >= head_num and (qkv_head_num - head_num) % 2 == 0,
            "packed head count must be head_num + 2 * kv_head_num")
    kv_head_num = (qkv_head_num - head_num) // 2
    _dev(qkv_buf)
    fn = getattr(capi.lib(), "isp_rope_decode_" + _suffix(qkv_buf))
    capi.check(fn(_p(qkv_buf), batch, head_num, kv_head_num, head_size, int(step), int(rotary_embedding_dim),
                  float(rotary_embedding_base), _stream()), "isp_rope_decode")
    return qkv_buf


def rope_decode_and_append(qkv_buf, qkv_bias, k_cache, v_cache, layer_id, history_length, step, head_num,
                           rotary_embedding_dim, rotary_embedding_base):
    """One decode step's bias + rotate-half RoPE + KV-cache append in a single launch: in place on qkv_buf
    [batch, head_num + 2 kv_head_num, head_size] at timestep step - 1 (as launchRoPE), and the rotated k row and
    the v row of sequence b go to cache[layer][b, head, history_length[b], :] (as launchConcatKVCache with one
    query token).  qkv_bias may be None.  step = 0: every sequence is rotated at its own history_length[b] instead
    (a batch whose sequences have different histories)."""
    _same_dtype(qkv_buf, qkv_bias, k_cache, v_cache)
    _int32(history_length)
    _expect(qkv_buf.dim() == 3, "qkv_buf must be [batch, heads, head_size]")
    batch, qkv_head_num, head_size = qkv_buf.shape
    _expect(qkv_head_num >= head_num and (qkv_head_num - head_num) % 2 == 0,
            "packed head count must be head_num + 2 * kv_head_num")
    kv_head_num = (qkv_head_num - head_num) // 2
    _expect(qkv_bias is None or qkv_bias.numel() == qkv_head_num * head_size,
            "qkv_bias must hold one value per packed column")
    _expect(k_cache.dim() == 5 and tuple(k_cache.shape) == tuple(v_cache.shape) and
            tuple(k_cache.shape[1:3]) == (batch, kv_head_num) and k_cache.shape[4] == head_size,
            "caches must be [layers, batch, kv_head_num, max_seq_len, head_size]")
    _expect(0 <= int(layer_id) < k_cache.shape[0], "layer_id outside the cache")
    _expect(history_length.numel() >= batch, "history_length is shorter than the batch")
    _dev(qkv_buf, qkv_bias, k_cache, v_cache, history_length)
    fn = getattr(capi.lib(), "isp_rope_decode_append_" + _suffix(qkv_buf))
    capi.check(fn(_p(qkv_buf), _p(qkv_bias), _p(k_cache), _p(v_cache), int(layer_id), k_cache.shape[3],
                  _p(history_length), batch, head_num, kv_head_num, head_size, int(step), int(rotary_embedding_dim),
                  float(rotary_embedding_base), _stream()), "isp_rope_decode_append")
    return qkv_buf, k_cache, v_cache


def transpose_out_remove_padding(qkv_buf_w_pad, padding_offset, qkv_buf_wo_pad):
    """launchTransposeOutRemovePadding: [batch, heads, seq, hs] -> [tokens, heads, hs]."""
    _same_dtype(qkv_buf_w_pad, qkv_buf_wo_pad)
    _int32(padding_offset)
    _expect(qkv_buf_w_pad.dim() == 4 and qkv_buf_wo_pad.dim() == 3,
            "transpose-out takes [batch, heads, seq, head_size] and [tokens, heads, head_size]")
    batch, head_num, seq_len, head_size = qkv_buf_w_pad.shape
    token_num = qkv_buf_wo_pad.shape[0]
    _expect(tuple(qkv_buf_wo_pad.shape[1:]) == (head_num, head_size), "packed output must be [tokens, heads, head_size]")
    _expect(padding_offset.numel() >= token_num, "padding_offset is shorter than the token count")
    _dev(qkv_buf_w_pad, padding_offset, qkv_buf_wo_pad)
    fn = getattr(capi.lib(), "isp_transpose_remove_padding_" + _suffix(qkv_buf_w_pad))
    capi.check(fn(_p(qkv_buf_w_pad), _p(padding_offset), _p(qkv_buf_wo_pad), batch, head_num, seq_len, head_size,
                  token_num, _stream()), "isp_transpose_remove_padding")
    return qkv_buf_wo_pad


def concat_kv_cache(k_src, v_src, layer_id, cur_query_length, history_length, k_dst, v_dst):
    """launchConcatKVCache; shapes as the reference derives them (concat_past_kv.cu:84-90)."""
    _same_dtype(k_src, v_src, k_dst, v_dst)
    _int32(cur_query_length, history_length)
    _expect(k_src.dim() == 4 and tuple(k_src.shape) == tuple(v_src.shape),
            "k_src and v_src must be [batch, kv_head_num, max_q_len, head_size]")
    batch, kv_head_num, max_q_len, head_size = k_src.shape
    _expect(k_dst.dim() == 5 and tuple(k_dst.shape) == tuple(v_dst.shape) and
            tuple(k_dst.shape[1:3]) == (batch, kv_head_num) and k_dst.shape[4] == head_size,
            "caches must be [layers, batch, kv_head_num, max_seq_len, head_size]")
    _expect(0 <= int(layer_id) < k_dst.shape[0], "layer_id outside the cache")
    _expect(cur_query_length.numel() >= batch and history_length.numel() >= batch,
            "length tensors are shorter than the batch")
    max_seq_len = k_dst.shape[3]
    _dev(k_src, v_src, cur_query_length, history_length, k_dst, v_dst)
    fn = getattr(capi.lib(), "isp_concat_kv_cache_" + _suffix(k_src))
    capi.check(fn(_p(k_src), _p(v_src), _p(k_dst), _p(v_dst), int(layer_id), _p(cur_query_length),
                  _p(history_length), batch, kv_head_num, max_q_len, max_seq_len, head_size, _stream()),
               "isp_concat_kv_cache")
    return k_dst, v_dst


def repeat_kv_cache(k_cache_src, v_cache_src, context_length, layer_id, k_cache_dst, v_cache_dst):
    """launchRepeatKVCache; shapes as the reference derives them (repeat_kv.cu:59-70)."""
    _same_dtype(k_cache_src, v_cache_src, k_cache_dst, v_cache_dst)
    _int32(context_length)
    _expect(k_cache_src.dim() == 5 and tuple(k_cache_src.shape) == tuple(v_cache_src.shape),
            "caches must be [layers, batch, kv_head_num, max_seq_len, head_size]")
    _expect(k_cache_dst.dim() == 4 and tuple(k_cache_dst.shape) == tuple(v_cache_dst.shape),
            "destinations must be [batch, head_num, max_k_len, head_size]")
    batch = context_length.shape[0]
    kv_head_num, max_seq_len = k_cache_src.shape[2], k_cache_src.shape[3]
    head_num, max_k_len, head_size = k_cache_dst.shape[1], k_cache_dst.shape[2], k_cache_dst.shape[3]
    _expect(k_cache_src.shape[1] == batch and k_cache_dst.shape[0] == batch, "batch extents differ")
    _expect(k_cache_src.shape[4] == head_size, "head sizes differ")
    _expect(kv_head_num > 0 and head_num % kv_head_num == 0, "head_num must be a multiple of kv_head_num")
    _expect(0 <= int(layer_id) < k_cache_src.shape[0], "layer_id outside the cache")
    _dev(k_cache_src, v_cache_src, context_length, k_cache_dst, v_cache_dst)
    fn = getattr(capi.lib(), "isp_repeat_kv_cache_" + _suffix(k_cache_src))
    capi.check(fn(_p(k_cache_src), _p(v_cache_src), _p(k_cache_dst), _p(v_cache_dst), int(layer_id),
                  _p(context_length), batch, head_num, kv_head_num, max_seq_len, max_k_len, head_size, _stream()),
               "isp_repeat_kv_cache")
    return k_cache_dst, v_cache_dst
