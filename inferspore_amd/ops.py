"""The C ABI called on torch tensors (device memory and the current stream come from torch).

Names and argument meaning mirror the reference's `launch*` functions; shapes are derived from the
tensors exactly as the reference's launchers derive them from `TensorWrapper::shape`.  All calls are
asynchronous on torch's current stream.  Nothing here computes on the host.
"""
import torch

from . import capi

_SUFFIX = {torch.float16: "f16", torch.float32: "f32"}


def _suffix(t):
    try:
        return _SUFFIX[t.dtype]
    except KeyError:
        raise TypeError("inferspore_amd kernels take float16 or float32 tensors, got %s" % t.dtype)


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
    _dev(input_ids, output, embed_table)
    if input_ids.dtype != torch.int32:
        raise TypeError("input_ids must be int32")
    if output.shape[0] != input_ids.shape[0]:
        raise RuntimeError("input ids 1st shape should equal to 1st shape of output")
    if output.dtype != embed_table.dtype:
        raise TypeError("output and table dtypes differ")
    fn = getattr(capi.lib(), "isp_embedding_" + _suffix(output))
    vocab = embed_table.shape[0] if check_bounds else 0
    capi.check(fn(_p(input_ids), _p(output), _p(embed_table), output.shape[0], output.shape[1],
                  vocab, _stream()), "isp_embedding")
    return output


def cal_padding_offset(padding_offset, cum_seqlens, input_lengths):
    """launchCalPaddingoffset: padding_offset [batch, max_q_len], cum_seqlens [batch + 1]."""
    _dev(padding_offset, cum_seqlens, input_lengths)
    batch, max_q_len = padding_offset.shape
    if batch != input_lengths.shape[0]:
        raise RuntimeError("input lenghts numbers should equal to padding offset bs dim!")
    if batch != cum_seqlens.shape[0] - 1:
        raise RuntimeError("cum seqlen numbers should equal to padding offset bs dim + 1!")
    for t in (padding_offset, cum_seqlens, input_lengths):
        if t.dtype != torch.int32:
            raise TypeError("padding-offset tensors must be int32")
    capi.check(capi.lib().isp_cal_padding_offset(_p(padding_offset), _p(cum_seqlens),
                                                 _p(input_lengths), batch, max_q_len, _stream()),
               "isp_cal_padding_offset")
    return padding_offset, cum_seqlens


def rmsnorm(x, gamma, eps):
    """In-place RMSNorm of x [tokens, hidden]."""
    _dev(x, gamma)
    _same_dtype(x, gamma)
    fn = getattr(capi.lib(), "isp_rmsnorm_" + _suffix(x))
    capi.check(fn(_p(x), _p(gamma), float(eps), x.shape[0], x.shape[1], _stream()), "isp_rmsnorm")
    return x


def fused_add_bias_residual_rmsnorm(residual, decoder_out, bias, gamma, eps, flags=0):
    """launchFusedAddBiasResidualRMSNorm: in place on residual (may be None) and decoder_out."""
    _dev(residual, decoder_out, bias, gamma)
    _same_dtype(decoder_out, residual, bias, gamma)
    fn = getattr(capi.lib(), "isp_fused_add_bias_residual_rmsnorm_" + _suffix(decoder_out))
    capi.check(fn(_p(residual), _p(decoder_out), _p(bias), _p(gamma), float(eps),
                  decoder_out.shape[0], decoder_out.shape[1], int(flags), _stream()),
               "isp_fused_add_bias_residual_rmsnorm")
    return residual, decoder_out


def add_fused_qkv_bias_transpose_and_rope(q_buf, k_buf, v_buf, qkv, qkv_bias, padding_offset,
                                          history_length, input_length, rotary_embedding_dim,
                                          rotary_embedding_base, max_position_embeddings=2048,
                                          use_dynamic_ntk=False):
    """launchAddFusedQKVBiasTransposeAndRoPE; shapes as the reference derives them
    (qkv_bias_and_RoPE.cu:298-304)."""
    _dev(q_buf, k_buf, v_buf, qkv, qkv_bias, padding_offset, history_length, input_length)
    _same_dtype(qkv, q_buf, k_buf, v_buf, qkv_bias)
    _int32(padding_offset, history_length, input_length)
    token_num, qkv_head_num, head_size = qkv.shape
    batch, head_num, seq_len = q_buf.shape[0], q_buf.shape[1], q_buf.shape[2]
    kv_head_num = (qkv_head_num - head_num) // 2
    fn = getattr(capi.lib(), "isp_qkv_bias_rope_transpose_" + _suffix(qkv))
    capi.check(fn(_p(q_buf), _p(k_buf), _p(v_buf), _p(qkv), _p(qkv_bias), _p(padding_offset),
                  _p(history_length), _p(input_length), batch, seq_len, token_num, head_num,
                  kv_head_num, head_size, int(rotary_embedding_dim), float(rotary_embedding_base),
                  int(max_position_embeddings), int(bool(use_dynamic_ntk)), _stream()),
               "isp_qkv_bias_rope_transpose")
    return q_buf, k_buf, v_buf


def act(input, out):
    """launchAct (SwiGLU): input [tokens, 2, inter] -> out [tokens, inter]."""
    _dev(input, out)
    _same_dtype(input, out)
    if input.shape[1] != 2:
        raise RuntimeError("SwiGLU input must have shape [tokens, 2, inter]")
    fn = getattr(capi.lib(), "isp_swiglu_" + _suffix(input))
    capi.check(fn(_p(input), _p(out), input.shape[0], input.shape[2], _stream()), "isp_swiglu")
    return out


def rope(qkv_buf, step, head_num, rotary_embedding_dim, rotary_embedding_base):
    """launchRoPE (decode): in place on qkv_buf [batch, head_num + 2 kv_head_num, head_size]; `step` is a
    host integer (the reference reads it from a CPU tensor)."""
    _dev(qkv_buf)
    batch, qkv_head_num, head_size = qkv_buf.shape
    kv_head_num = (qkv_head_num - head_num) // 2
    fn = getattr(capi.lib(), "isp_rope_decode_" + _suffix(qkv_buf))
    capi.check(fn(_p(qkv_buf), batch, head_num, kv_head_num, head_size, int(step), int(rotary_embedding_dim),
                  float(rotary_embedding_base), _stream()), "isp_rope_decode")
    return qkv_buf


def transpose_out_remove_padding(qkv_buf_w_pad, padding_offset, qkv_buf_wo_pad):
    """launchTransposeOutRemovePadding: [batch, heads, seq, hs] -> [tokens, heads, hs]."""
    _dev(qkv_buf_w_pad, padding_offset, qkv_buf_wo_pad)
    _same_dtype(qkv_buf_w_pad, qkv_buf_wo_pad)
    _int32(padding_offset)
    batch, head_num, seq_len, head_size = qkv_buf_w_pad.shape
    token_num = qkv_buf_wo_pad.shape[0]
    fn = getattr(capi.lib(), "isp_transpose_remove_padding_" + _suffix(qkv_buf_w_pad))
    capi.check(fn(_p(qkv_buf_w_pad), _p(padding_offset), _p(qkv_buf_wo_pad), batch, head_num, seq_len, head_size,
                  token_num, _stream()), "isp_transpose_remove_padding")
    return qkv_buf_wo_pad


def concat_kv_cache(k_src, v_src, layer_id, cur_query_length, history_length, k_dst, v_dst):
    """launchConcatKVCache; shapes as the reference derives them (concat_past_kv.cu:84-90)."""
    _dev(k_src, v_src, cur_query_length, history_length, k_dst, v_dst)
    _same_dtype(k_src, v_src, k_dst, v_dst)
    _int32(cur_query_length, history_length)
    batch, kv_head_num, max_q_len, head_size = k_src.shape
    max_seq_len = k_dst.shape[3]
    fn = getattr(capi.lib(), "isp_concat_kv_cache_" + _suffix(k_src))
    capi.check(fn(_p(k_src), _p(v_src), _p(k_dst), _p(v_dst), int(layer_id), _p(cur_query_length),
                  _p(history_length), batch, kv_head_num, max_q_len, max_seq_len, head_size, _stream()),
               "isp_concat_kv_cache")
    return k_dst, v_dst


def repeat_kv_cache(k_cache_src, v_cache_src, context_length, layer_id, k_cache_dst, v_cache_dst):
    """launchRepeatKVCache; shapes as the reference derives them (repeat_kv.cu:59-70)."""
    _dev(k_cache_src, v_cache_src, context_length, k_cache_dst, v_cache_dst)
    _same_dtype(k_cache_src, v_cache_src, k_cache_dst, v_cache_dst)
    _int32(context_length)
    batch = context_length.shape[0]
    kv_head_num, max_seq_len = k_cache_src.shape[2], k_cache_src.shape[3]
    head_num, max_k_len, head_size = k_cache_dst.shape[1], k_cache_dst.shape[2], k_cache_dst.shape[3]
    fn = getattr(capi.lib(), "isp_repeat_kv_cache_" + _suffix(k_cache_src))
    capi.check(fn(_p(k_cache_src), _p(v_cache_src), _p(k_cache_dst), _p(v_cache_dst), int(layer_id),
                  _p(context_length), batch, head_num, kv_head_num, max_seq_len, max_k_len, head_size, _stream()),
               "isp_repeat_kv_cache")
    return k_cache_dst, v_cache_dst
