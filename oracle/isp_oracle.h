/*
 * isp_oracle.h -- CPU oracle for the InferSpore fused per-layer kernels.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP kernels are
 * compared against (tests, the smoke check, and the cpu_baseline leg of the
 * benchmark).  Nothing that ships as the product links, loads or calls it.
 *
 * Every function is a plain-C restatement of the algorithm the reference
 * implements for that step; the comment on each names the reference lines it
 * follows and every place where the restatement deliberately departs from a
 * defect in the reference.
 *
 * fp16 tensors are passed as uint16_t bit patterns (IEEE binary16); all fp16
 * arithmetic is "convert to fp32, compute in fp32, round once (nearest-even)".
 *
 * Pinning status (what independent evidence fixes each function; the tests
 * under tests/test_oracle_*.py hold the checks):
 *   isp_oracle_h2f / f2h            exhaustive / randomised vs numpy.float16
 *   isp_oracle_embedding            reference known answer table[r,:]=r  +  numpy take
 *   isp_oracle_cal_padding_offset   reference known answer (3,3,3 / max 5)  +  numpy cumsum
 *   isp_oracle_fused_norm_*         reference known answer 1/sqrt(1.5)  +  float64 closed form,
 *                                   invariants (scale equivariance, residual identity)
 *   isp_oracle_qkv_rope_*           reference known answer 32(cos -/+ sin)  +  float64 textbook
 *                                   rotation, norm invariance, t=0 identity, brute-force scatter
 *   isp_oracle_swiglu_*             reference known answer 0.7310586  +  float64 closed form,
 *                                   silu(x)-silu(-x)=x
 *   isp_oracle_rope_decode_*        float64 textbook rotation, equality with the prefill step at
 *                                   history=step-1
 *   isp_oracle_transpose_remove_padding   reference layout example  +  inverse of the qkv scatter
 *   isp_oracle_concat_kv / repeat_kv      brute-force numpy slicing
 */
#ifndef ISP_ORACLE_H
#define ISP_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* flag for the fused norm: reproduce the reference fp32 kernel literally, i.e.
 * store residual := residual + out and add the bias only afterwards
 * (fused_addresidual_norm.cu:56-73).  Default (0) stores residual + out + bias. */
#define ISP_ORACLE_NORM_RESIDUAL_EXCLUDES_BIAS 1u

/* number of OpenMP threads the row loops use (1 = serial, as the reference's
 * CPU loops are written).  Returns the value now in effect. */
int isp_oracle_set_threads(int n);
int isp_oracle_max_threads(void);

/* IEEE binary16 <-> binary32, round-to-nearest-even. */
float    isp_oracle_h2f(uint16_t h);
uint16_t isp_oracle_f2h(float f);
void     isp_oracle_h2f_array(const uint16_t* h, float* f, size_t n);
void     isp_oracle_f2h_array(const float* f, uint16_t* h, size_t n);

/* out[t, :] = table[ids[t], :]; elem_size = bytes per element (2 or 4). */
void isp_oracle_embedding(const int32_t* ids, void* out, const void* table,
                          int tokens, int hidden, int elem_size);

void isp_oracle_cal_padding_offset(int32_t* padding_offset, int32_t* cum_seqlens,
                                   const int32_t* input_lengths, int batch, int max_q_len);

/* residual / bias may be NULL.  In place on residual and decoder_out. */
void isp_oracle_fused_norm_f32(float* residual, float* decoder_out, const float* bias,
                               const float* gamma, float eps, int tokens, int hidden,
                               unsigned flags);
void isp_oracle_fused_norm_f16(uint16_t* residual, uint16_t* decoder_out, const uint16_t* bias,
                               const uint16_t* gamma, float eps, int tokens, int hidden,
                               unsigned flags);

/* q [batch, head_num, seq_len, head_size], k/v [batch, kv_head_num, seq_len, head_size];
 * qkv [token_num, head_num + 2 kv_head_num, head_size]; bias may be NULL. */
void isp_oracle_qkv_rope_f32(float* q, float* k, float* v, const float* qkv, const float* bias,
                             const int32_t* padding_offset, const int32_t* history_length,
                             const int32_t* input_length, int batch, int seq_len, int token_num,
                             int head_num, int kv_head_num, int head_size, int rotary_dim,
                             float rotary_base);
void isp_oracle_qkv_rope_f16(uint16_t* q, uint16_t* k, uint16_t* v, const uint16_t* qkv,
                             const uint16_t* bias, const int32_t* padding_offset,
                             const int32_t* history_length, const int32_t* input_length,
                             int batch, int seq_len, int token_num, int head_num,
                             int kv_head_num, int head_size, int rotary_dim, float rotary_base);

/* in [tokens, 2, inter], out [tokens, inter]. */
void isp_oracle_swiglu_f32(const float* in, float* out, int tokens, int inter);
void isp_oracle_swiglu_f16(const uint16_t* in, uint16_t* out, int tokens, int inter);

/* decode-phase RoPE, in place on a packed qkv row [batch, head_num + 2 kv_head_num, head_size]. */
void isp_oracle_rope_decode_f32(float* qkv, int batch, int head_num, int kv_head_num,
                                int head_size, int step, int rotary_dim, float rotary_base);
void isp_oracle_rope_decode_f16(uint16_t* qkv, int batch, int head_num, int kv_head_num,
                                int head_size, int step, int rotary_dim, float rotary_base);

/* [batch, head_num, seq_len, head_size] -> [token_num, head_num, head_size]. */
void isp_oracle_transpose_remove_padding(const void* src, void* dst, const int32_t* padding_offset,
                                         int batch, int head_num, int seq_len, int head_size,
                                         int token_num, int elem_size);

/* src [batch, kv_head_num, max_q_len, head_size] -> cache layer
 * [batch, kv_head_num, max_seq_len, head_size] at rows history[b] .. history[b]+cur_len[b]. */
void isp_oracle_concat_kv(const void* src, void* cache, size_t layer_offset_elems,
                          const int32_t* cur_query_length, const int32_t* history_length,
                          int batch, int kv_head_num, int max_q_len, int max_seq_len,
                          int head_size, int elem_size);

/* cache layer [batch, kv_head_num, max_seq_len, head_size] -> dst [batch, head_num, max_k_len, head_size]. */
void isp_oracle_repeat_kv(const void* cache, void* dst, size_t layer_offset_elems,
                          const int32_t* context_length, int batch, int head_num, int kv_head_num,
                          int max_seq_len, int max_k_len, int head_size, int elem_size);

#ifdef __cplusplus
}
#endif
#endif
