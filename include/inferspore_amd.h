/*
 * inferspore_amd.h -- C ABI of the MI355X (gfx950) implementation of InferSpore's fused
 * per-layer kernels.
 *
 * This is the drop-in boundary: every entry point takes raw device pointers, plain integers and a
 * HIP stream, launches hand-written HIP kernels asynchronously on that stream, allocates nothing
 * and returns 0 or a negative isp_status.  The library keeps no state between calls except the
 * process-wide tuning knobs of isp_tuning_set (atomic; they select among kernel variants with
 * identical results, and nothing sets them unless the caller does).  The C++ `launch*` templates declared
 * under include/src/kernels/ (same names and parameter lists as the reference's) are thin shims
 * over these functions; a binding from any other language needs only this header.
 *
 * Each declaration names the reference interface it replaces (paths relative to the
 * m0dulo/InferSpore checkout).
 *
 * Conventions
 *   - all tensors are dense, row-major, device-resident; `_f16` = IEEE binary16 storage with fp32
 *     arithmetic and a single rounding per stored value, `_f32` = binary32 throughout;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream, which is what the
 *     reference's launchers use);
 *   - pointers documented "may be NULL" are optional operands; any other NULL pointer gives
 *     ISP_ERR_NULL_POINTER (unless the call has no work to do: zero tokens returns ISP_OK first);
 *   - 16-byte aligned pointers and vector-friendly extents take the fast 128-bit path; anything
 *     else is routed to a slower scalar kernel with identical results.  Tensor pointers must be
 *     aligned to their element (2 bytes for `_f16`, 4 for `_f32`, 4 for the int32 arrays); the
 *     pure movers (gather, transpose-out, KV append / broadcast) accept any byte address;
 */
#ifndef INFERSPORE_AMD_H
#define INFERSPORE_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum isp_status {
    ISP_OK = 0,
    ISP_ERR_NULL_POINTER = -1, /* a required pointer is NULL */
    ISP_ERR_BAD_SHAPE = -2,    /* negative / inconsistent extents */
    ISP_ERR_UNSUPPORTED = -3,  /* extents outside what the kernels implement */
    ISP_ERR_LAUNCH = -4,       /* HIP reported an error at launch; see isp_last_hip_error() */
    ISP_ERR_DEVICE = -5        /* no usable gfx950 device */
} isp_status;

/* flag bits for isp_fused_add_bias_residual_rmsnorm_* */
#define ISP_NORM_RESIDUAL_EXCLUDES_BIAS 1u

typedef void* isp_stream_t; /* hipStream_t */

/* Library identification and diagnostics (no reference counterpart). */
const char* isp_version(void);
const char* isp_strerror(int status);
/* hipError_t of the most recent failed launch on the calling thread (0 if none). */
int isp_last_hip_error(void);
/* Checks that the current HIP device exists and is a gfx950; optional, the kernels need no set-up. */
int isp_init(void);

/*
 * Input-embedding gather: out[t, :] = table[ids[t], :].
 * Replaces launchInputEmbedding<T> (src/kernels/input_embedding.h:6-9, .cu:25-45).
 *   ids [tokens] int32, table [vocab, hidden], out [tokens, hidden].
 * `vocab` > 0 enables a bounds check (rows whose id is outside [0, vocab) are written as zeros
 * instead of reading out of bounds); vocab == 0 reproduces the reference's unchecked gather.
 */
int isp_embedding_f16(const int32_t* ids, void* out, const void* table, int tokens, int hidden,
                      int vocab, isp_stream_t stream);
int isp_embedding_f32(const int32_t* ids, void* out, const void* table, int tokens, int hidden,
                      int vocab, isp_stream_t stream);

/*
 * Padding-offset builder.
 * Replaces launchCalPaddingoffset (src/kernels/cal_paddingoffset.h:8-11, .cu:18-60).
 *   input_lengths [batch]; padding_offset [batch, max_q_len] (only the first sum(lengths) entries
 *   are written); cum_seqlens [batch + 1].
 */
int isp_cal_padding_offset(int32_t* padding_offset, int32_t* cum_seqlens,
                           const int32_t* input_lengths, int batch, int max_q_len,
                           isp_stream_t stream);

/*
 * RMSNorm, in place: x := x * rsqrt(mean(x^2) + eps) * gamma.
 * The reference reaches this through launchFusedAddBiasResidualRMSNorm<T> with a NULL residual and
 * bias (src/kernels/fused_addresidual_norm.cu:51,56,68); same kernel here.
 *   x [tokens, hidden], gamma [hidden].
 */
int isp_rmsnorm_f32(void* x, const void* gamma, float eps, int tokens, int hidden,
                    isp_stream_t stream);
int isp_rmsnorm_f16(void* x, const void* gamma, float eps, int tokens, int hidden,
                    isp_stream_t stream);

/*
 * Fused add-bias + residual + RMSNorm, in place on both tensors.
 * Replaces launchFusedAddBiasResidualRMSNorm<T> (src/kernels/fused_addresidual_norm.h:9-15,
 * .cu:32-98,143-170).
 *   x            = decoder_out + residual + bias
 *   residual    := x                       (flags == 0)
 *   residual    := decoder_out + residual  (ISP_NORM_RESIDUAL_EXCLUDES_BIAS: the reference's
 *                                           literal store order, .cu:62-67)
 *   decoder_out := gamma * x * rsqrt(mean(x^2) + eps)
 *   residual, decoder_out [tokens, hidden]; bias, gamma [hidden]; residual and bias may be NULL.
 *   residual and decoder_out must be distinct buffers (each is read and written once).
 */
int isp_fused_add_bias_residual_rmsnorm_f32(void* residual, void* decoder_out, const void* bias,
                                            const void* gamma, float eps, int tokens, int hidden,
                                            unsigned flags, isp_stream_t stream);
int isp_fused_add_bias_residual_rmsnorm_f16(void* residual, void* decoder_out, const void* bias,
                                            const void* gamma, float eps, int tokens, int hidden,
                                            unsigned flags, isp_stream_t stream);

/*
 * Fused QKV bias + rotate-half RoPE + head transpose + re-padding (prefill).
 * Replaces launchAddFusedQKVBiasTransposeAndRoPE<T> (src/kernels/qkv_bias_and_RoPE.h:10-20,
 * .cu:109-192,286-330).
 *   qkv [token_num, head_num + 2 kv_head_num, head_size] packed (no padding);
 *   bias [(head_num + 2 kv_head_num) * head_size], may be NULL;
 *   padding_offset [token_num]; history_length, input_length [batch];
 *   q [batch, head_num, seq_len, head_size]; k, v [batch, kv_head_num, seq_len, head_size].
 * Token t lands at flat padded position p = t + padding_offset[t] (b = p / seq_len,
 * s = p % seq_len) and is rotated at timestep history_length[b] + s.  Padded positions are not
 * written.  A token whose p falls outside [0, batch * seq_len) is skipped (the reference would
 * write out of bounds).  `max_position_embeddings` and `use_dynamic_ntk` are accepted and ignored,
 * as in the reference (.cu:126-127).  The outputs must not overlap the input.
 * head_size must be even, rotary_embedding_dim even and <= min(head_size, 256).
 */
int isp_qkv_bias_rope_transpose_f32(void* q, void* k, void* v, const void* qkv, const void* bias,
                                    const int32_t* padding_offset, const int32_t* history_length,
                                    const int32_t* input_length, int batch, int seq_len,
                                    int token_num, int head_num, int kv_head_num, int head_size,
                                    int rotary_embedding_dim, float rotary_embedding_base,
                                    int max_position_embeddings, int use_dynamic_ntk,
                                    isp_stream_t stream);
int isp_qkv_bias_rope_transpose_f16(void* q, void* k, void* v, const void* qkv, const void* bias,
                                    const int32_t* padding_offset, const int32_t* history_length,
                                    const int32_t* input_length, int batch, int seq_len,
                                    int token_num, int head_num, int kv_head_num, int head_size,
                                    int rotary_embedding_dim, float rotary_embedding_base,
                                    int max_position_embeddings, int use_dynamic_ntk,
                                    isp_stream_t stream);

/*
 * The same step with the KV-cache append fused in: besides (k, v non-NULL) or instead of (k, v both
 * NULL) the padded k / v buffers, the k and v rows of token (b, s) are written to
 *   cache[layer][b, head, history_length[b] + s, :]      when s < input_length[b]
 * (rows that would fall outside [0, max_seq_len) are skipped), i.e. what launchConcatKVCache<T>
 * (src/kernels/concat_past_kv.h:7-14, .cu:7-113) does in a second pass over k and v with
 * cur_query_length = input_length.  The results are the bits of isp_qkv_bias_rope_transpose_*
 * followed by isp_concat_kv_cache_*; one launch and one HBM pass less (with k, v NULL the k / v rows
 * are written once instead of written, re-read and written again).
 *   k_cache, v_cache [layers, batch, kv_head_num, max_seq_len, head_size] (base pointers).
 * Extends launchAddFusedQKVBiasTransposeAndRoPE<T> (src/kernels/qkv_bias_and_RoPE.h:10-20); the
 * reference has no fused form.
 */
int isp_qkv_bias_rope_transpose_append_f32(void* q, void* k, void* v, void* k_cache, void* v_cache,
                                           int layer, int max_seq_len, const void* qkv,
                                           const void* bias, const int32_t* padding_offset,
                                           const int32_t* history_length,
                                           const int32_t* input_length, int batch, int seq_len,
                                           int token_num, int head_num, int kv_head_num,
                                           int head_size, int rotary_embedding_dim,
                                           float rotary_embedding_base, isp_stream_t stream);
int isp_qkv_bias_rope_transpose_append_f16(void* q, void* k, void* v, void* k_cache, void* v_cache,
                                           int layer, int max_seq_len, const void* qkv,
                                           const void* bias, const int32_t* padding_offset,
                                           const int32_t* history_length,
                                           const int32_t* input_length, int batch, int seq_len,
                                           int token_num, int head_num, int kv_head_num,
                                           int head_size, int rotary_embedding_dim,
                                           float rotary_embedding_base, isp_stream_t stream);

/*
 * SwiGLU activation: out[t, i] = silu(in[t, 0, i]) * in[t, 1, i], silu(x) = x / (1 + exp(-x)).
 * Replaces launchAct<T> (src/kernels/act_kernel.h:8-9, .cu:18-71).
 *   in [tokens, 2, inter], out [tokens, inter].
 */
int isp_swiglu_f32(const void* in, void* out, int tokens, int inter, isp_stream_t stream);
int isp_swiglu_f16(const void* in, void* out, int tokens, int inter, isp_stream_t stream);

/*
 * Decode-phase RoPE, in place: rotate-half on the q and k heads of packed rows
 * [batch, head_num + 2 kv_head_num, head_size] at timestep step - 1 (step >= 1).
 * Replaces launchRoPE<T> (src/kernels/qkv_bias_and_RoPE.h:22-25, .cu:352-434; the reference's fp16
 * body is empty and its launcher only accepts batch 1, 32+32+32 heads of 128).
 */
int isp_rope_decode_f32(void* qkv, int batch, int head_num, int kv_head_num, int head_size, int step,
                        int rotary_embedding_dim, float rotary_embedding_base, isp_stream_t stream);
int isp_rope_decode_f16(void* qkv, int batch, int head_num, int kv_head_num, int head_size, int step,
                        int rotary_embedding_dim, float rotary_embedding_base, isp_stream_t stream);

/*
 * Fused decode step: QKV bias (may be NULL) + rotate-half RoPE at timestep step - 1, in place on the
 * packed rows as isp_rope_decode_*, and the KV-cache append of the one new token per sequence:
 *   k_cache[layer][b, head, history_length[b], :] = rotated k row,  v_cache[...] = v row
 * (rows outside [0, max_seq_len) are skipped).  With the bias the v heads are updated in place too.
 * One launch for launchRoPE<T> (src/kernels/qkv_bias_and_RoPE.cu:352-434) followed by
 * launchConcatKVCache<T> with a one-token query (src/kernels/concat_past_kv.cu:7-113), whose results
 * it reproduces bit for bit; each of the two is launch-bound alone.  The reference has no fused form
 * outside its attention kernel (src/kernels/fused_decoder_self_attention.cu:162-200).
 * The one timestep step - 1 for the whole batch is the reference's launchRoPE (which only accepts batch 1);
 * it agrees with the row the append writes only where history_length[b] == step - 1.  For a batch whose
 * sequences have different histories pass step = 0: every sequence is then rotated at its own
 * history_length[b], the position its row is appended at (= the prefill kernel on one-token sequences).
 */
int isp_rope_decode_append_f32(void* qkv, const void* bias, void* k_cache, void* v_cache, int layer,
                               int max_seq_len, const int32_t* history_length, int batch,
                               int head_num, int kv_head_num, int head_size, int step,
                               int rotary_embedding_dim, float rotary_embedding_base,
                               isp_stream_t stream);
int isp_rope_decode_append_f16(void* qkv, const void* bias, void* k_cache, void* v_cache, int layer,
                               int max_seq_len, const int32_t* history_length, int batch,
                               int head_num, int kv_head_num, int head_size, int step,
                               int rotary_embedding_dim, float rotary_embedding_base,
                               isp_stream_t stream);

/*
 * Transpose attention output and remove padding: dst[t, h, :] = src[b, h, s, :] with
 * t + padding_offset[t] = b * seq_len + s.  src [batch, head_num, seq_len, head_size],
 * dst [token_num, head_num, head_size].
 * Supplies launchTransposeOutRemovePadding<T>, which the reference declares
 * (src/kernels/fused_transpose_and_remv_pad.h:7-10) and tests
 * (tests/unittests/test_fused_trans_remv_pad.cu) but does not define.
 */
int isp_transpose_remove_padding_f32(const void* src, const int32_t* padding_offset, void* dst,
                                     int batch, int head_num, int seq_len, int head_size,
                                     int token_num, isp_stream_t stream);
int isp_transpose_remove_padding_f16(const void* src, const int32_t* padding_offset, void* dst,
                                     int batch, int head_num, int seq_len, int head_size,
                                     int token_num, isp_stream_t stream);

/*
 * KV-cache append: cache[layer][b, h, history_length[b] + t, :] = src[b, h, t, :] for
 * t < cur_query_length[b], for k and v in one launch.
 * k_src, v_src [batch, kv_head_num, max_q_len, head_size];
 * k_cache, v_cache [layers, batch, kv_head_num, max_seq_len, head_size] (base pointers; `layer`
 * selects the slice).  Replaces launchConcatKVCache<T> (src/kernels/concat_past_kv.h:7-14,
 * .cu:7-113).
 */
int isp_concat_kv_cache_f32(const void* k_src, const void* v_src, void* k_cache, void* v_cache,
                            int layer, const int32_t* cur_query_length,
                            const int32_t* history_length, int batch, int kv_head_num, int max_q_len,
                            int max_seq_len, int head_size, isp_stream_t stream);
int isp_concat_kv_cache_f16(const void* k_src, const void* v_src, void* k_cache, void* v_cache,
                            int layer, const int32_t* cur_query_length,
                            const int32_t* history_length, int batch, int kv_head_num, int max_q_len,
                            int max_seq_len, int head_size, isp_stream_t stream);

/*
 * KV-cache broadcast to the query heads (GQA / MQA):
 * dst[b, h, s, :] = cache[layer][b, h / (head_num / kv_head_num), s, :] for s < context_length[b].
 * k_dst, v_dst [batch, head_num, max_k_len, head_size].
 * Replaces launchRepeatKVCache<T> (src/kernels/repeat_kv.h:7-13, .cu:10-100).
 */
int isp_repeat_kv_cache_f32(const void* k_cache, const void* v_cache, void* k_dst, void* v_dst,
                            int layer, const int32_t* context_length, int batch, int head_num,
                            int kv_head_num, int max_seq_len, int max_k_len, int head_size,
                            isp_stream_t stream);
int isp_repeat_kv_cache_f16(const void* k_cache, const void* v_cache, void* k_dst, void* v_dst,
                            int layer, const int32_t* context_length, int batch, int head_num,
                            int kv_head_num, int max_seq_len, int max_k_len, int head_size,
                            isp_stream_t stream);

/*
 * Measurement aids (no reference counterpart).
 * isp_calibration_copy: a plain copy kernel of known traffic (`bytes` read + `bytes` written;
 *   16-byte aligned, multiple of 16) used to calibrate profiler byte counters and to measure the
 *   copy bandwidth the machine actually reaches.
 * isp_tuning_set: overrides a launch heuristic process-wide (0 restores the automatic choice) and
 *   returns the previous value, or ISP_ERR_BAD_SHAPE for an unknown knob.  For benchmark sweeps;
 *   results never depend on the knobs, only speed does.  Thread-safe (each knob is an atomic that a
 *   launcher reads once per call); a serving process has no reason to call it.
 */
int isp_calibration_copy(void* dst, const void* src, size_t bytes, isp_stream_t stream);
/* isp_norm_launch_config: which instantiation isp_rmsnorm_* / isp_fused_add_bias_residual_rmsnorm_*
 *   launch for `tokens` rows of `hidden` elements of `elem_size` bytes (2 or 4) on the vector path
 *   (`fused` != 0: with a residual operand) -- waves per row, 16-byte vectors per lane, threads per
 *   workgroup and store kind (0 plain, 1 non-temporal, 2 write-through), i.e. the template arguments
 *   of isp::fused_norm_rows in a profiler trace.  Any output pointer may be NULL.  ISP_ERR_UNSUPPORTED
 *   when the shape takes the scalar kernel. */
int isp_norm_launch_config(int elem_size, int tokens, int hidden, int fused, int* waves_per_row,
                           int* vectors_per_lane, int* block_threads, int* store_kind);

/* isp_norm_launch_variant: 1 if a call with these operands (`flags` as for the fused entry point) is launched
 *   as isp::fused_norm_few_rows -- the same row algorithm with the operand set fixed at compile time, taken by
 *   launches whose waves are all resident at once (every decode-step norm, prefill batches of a few hundred
 *   rows) unless they want the general kernel's pacing load -- and 0 if as the general
 *   isp::fused_norm_rows; the waves per row, vectors per lane and store kind are those of
 *   isp_norm_launch_config, the workgroup is max(256, 64 x waves per row) threads.  No counterpart in the
 *   reference (its launcher has one configuration, src/kernels/fused_addresidual_norm.cu:155-159). */
int isp_norm_launch_variant(int elem_size, int tokens, int hidden, int has_residual, int has_bias, unsigned flags);

typedef enum isp_tuning_knob {
    ISP_TUNE_NORM_WAVES_PER_ROW = 0, /* 1, 2, 4, 8 or 16 waves cooperate on one token row */
    ISP_TUNE_NORM_STORE = 1,         /* output stores: 1 = plain (default where a launch writes at most 1 MiB),
                                        2 = non-temporal (default otherwise), 3 = non-temporal write-through */
    ISP_TUNE_SWIGLU_UNROLL = 2,      /* 1 (default), 2 or 4 vector pairs in flight per lane */
    ISP_TUNE_SWIGLU_STORE = 3,       /* 1 = plain, 2 = non-temporal (default), 3 = write-through */
    ISP_TUNE_EMBED_VARIANT = 4,      /* 1 = a wave per row, 2 = a workgroup per row,
                                        3 = a single-wave workgroup per 1 KiB chunk of a row (default) */
    ISP_TUNE_EMBED_STORE = 5,        /* 1 = plain (default up to 1 MiB of output), 2 = non-temporal (default up to
                                        8 MiB), 3 = write-through (default above) */
    ISP_TUNE_QKV_STORE = 6,          /* 1 = plain, 2 = non-temporal, 3 = write-through (default) */
    ISP_TUNE_QKV_WAVES = 7,          /* 1, 2 or 4: the general kernel with that many waves (groups of 8 heads) per
                                        workgroup; 8: as 0, but 64-element fp16 heads take the one-token whole-row
                                        kernel; 0 = automatic: the one-vector-per-lane kernels where the shape
                                        allows them (128-element heads fully rotated with head counts multiples of
                                        4 in fp16, of 2 in fp32; 64-element fp16 heads fully rotated with head
                                        counts multiples of 8), else the general kernel with 4 waves */
    ISP_TUNE_NORM_BLOCK_THREADS = 8, /* 256, 512 or 1024 threads per workgroup (several token rows share a
                                        workgroup when a row needs fewer); 0 = automatic */
    ISP_TUNE_NORM_ORDER = 9,         /* 2 = streaming (each vector processed, and the residual stored, as it
                                        arrives); 0, 1 = read everything, then write everything (default);
                                        3 = as 0, but launches of a few rows also take the general kernel;
                                        4 / 5 = as 0, but a call with a residual and no bias never / always waits
                                        for a gamma vector where the bias vector would arrive (by default it does
                                        where the launch is one round of waves reading more than 24 MiB) */
    ISP_TUNE_MOVER_BLOCK_THREADS = 10, /* KV append / broadcast: 64, 128, 256 (default), 512 or 1024 threads per
                                          workgroup; transpose-out: 64 (default), 128, 256 or 512 */
    ISP_TUNE_COUNT = 11
} isp_tuning_knob;
int isp_tuning_set(int knob, int value);

#ifdef __cplusplus
}
#endif
#endif /* INFERSPORE_AMD_H */
