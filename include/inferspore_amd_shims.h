/* Options of the C++ launch* shims (include/src/kernels/*.h).  Nothing here has a counterpart in the
 * reference; the C ABI (inferspore_amd.h) is not affected. */
#pragma once

namespace isp_shims {

/* How the shims treat the optional biases.
 *
 * false (the default): as the operators' names say.  launchFusedAddBiasResidualRMSNorm stores
 *   residual = residual + decoder_out + bias, and launchAddFusedQKVBiasTransposeAndRoPE (and the form
 *   with the KV append) adds qkv.bias before rotating.
 * true: what the reference's kernels literally do with a non-null bias.  The stored residual leaves the
 *   bias out (src/kernels/fused_addresidual_norm.cu:56-73: it is written before the bias is added, with a
 *   TODO saying so), and qkv.bias is never read (src/kernels/qkv_bias_and_RoPE.cu:141-160 has no bias
 *   add in the fp32 kernel, :228-252 has it commented out in the fp16 one).  For a model whose checkpoint
 *   carries attention biases (src/weights/llama/layer_weights.cc:28-57) this reproduces the reference's
 *   activations; with null biases, as LLaMA has, the two modes are identical.
 *
 * The initial value is taken once from the environment variable ISP_SHIMS_REFERENCE_LITERAL_BIAS
 * ("1" = true).  Process-wide and atomic; returns the previous setting. */
bool setReferenceLiteralBias(bool on);
bool referenceLiteralBias();

}  // namespace isp_shims
