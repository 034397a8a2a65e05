// RMSNorm and fused add-residual + RMSNorm for launches of a few rows -- every decode-step norm, and prefill
// batches up to the size whose waves are all resident at once -- on gfx950.
// Semantics and row algorithm: norm_rows.h (src/kernels/fused_addresidual_norm.cu:55-97 in the reference).
// This file is built with kernel-argument preloading like the other kernel files: the arguments arrive in scalar
// registers with the wave instead of being fetched by its first instructions, one round trip less in a launch
// that is nothing but a chain of round trips (64 x 4096 fp32: 2.40 against 2.64 us per launch; 256 rows 3.2
// against 3.4).  The general kernel (norm.hip) is built without it: the benchmark configuration, 2048 x 4096
// fp16 with residual and bias in one round of waves, measured 1 % slower with it.
#include "norm_rows.h"

namespace isp {

// The same row algorithm for launches of a few rows (every decode-step norm).  Such a launch is a chain of
// latencies, not a stream: the device is mostly empty, nothing hides an instruction, and what the general
// kernel pays for deciding at run time which operands exist and in which order to store (branches, selects,
// and waits that must assume the worst because loads sit inside branches) is on the critical path -- 64 x
// 4096 fp32: 2.9 us per launch back to back with the general kernel, 2.6 us with the operands fixed at
// compile time, 2.4 us with the arguments preloaded as well, against 2.0 us for a copy of the same bytes.  One row per workgroup of WPR waves, one or two
// vectors per lane, the default residual order only.  Same operations in the same order, so the same bits.
// (Requesting gamma and bias together with the row, to take a cache round trip out of the chain, measured
// 0.05-0.2 us SLOWER at 16-256 rows, twice, in this kernel and in a stripped-down one.)
template <typename T, int NV, int WPR, int ST, int OPS>
__global__ __launch_bounds__(norm_block(WPR)) void fused_norm_few_rows(T* residual, T* out, const T* bias,
                                                                       const T* gamma, float eps, int tokens,
                                                                       int hidden) {
    norm_rows_body<T, NV, WPR, ST, norm_block(WPR), OPS>(residual, out, bias, gamma, eps, tokens, hidden, 0u);
}

template <typename T, int NV, int WPR, int ST>
static NormFewKernel<T> few_ops(int ops) {
    if (ops == kOpsNone) return fused_norm_few_rows<T, NV, WPR, ST, kOpsNone>;
    if (ops == kOpsResidual) return fused_norm_few_rows<T, NV, WPR, ST, kOpsResidual>;
    return fused_norm_few_rows<T, NV, WPR, ST, kOpsResidualBias>;
}

template <typename T>
NormFewKernel<T> norm_few_variant(int wpr, int nv, int st, int ops) {
    if (st != kStorePlain && st != kStoreStream) return nullptr;
    const bool plain = st == kStorePlain;
    if (nv == 2 && wpr == 16)
        return plain ? few_ops<T, 2, 16, kStorePlain>(ops) : few_ops<T, 2, 16, kStoreStream>(ops);
    if (nv != 1) return nullptr;
    switch (wpr) {
        case 1: return plain ? few_ops<T, 1, 1, kStorePlain>(ops) : few_ops<T, 1, 1, kStoreStream>(ops);
        case 2: return plain ? few_ops<T, 1, 2, kStorePlain>(ops) : few_ops<T, 1, 2, kStoreStream>(ops);
        case 4: return plain ? few_ops<T, 1, 4, kStorePlain>(ops) : few_ops<T, 1, 4, kStoreStream>(ops);
        case 8: return plain ? few_ops<T, 1, 8, kStorePlain>(ops) : few_ops<T, 1, 8, kStoreStream>(ops);
        case 16: return plain ? few_ops<T, 1, 16, kStorePlain>(ops) : few_ops<T, 1, 16, kStoreStream>(ops);
        default: return nullptr;
    }
}

template NormFewKernel<float> norm_few_variant<float>(int, int, int, int);
template NormFewKernel<__half> norm_few_variant<__half>(int, int, int, int);

}  // namespace isp
