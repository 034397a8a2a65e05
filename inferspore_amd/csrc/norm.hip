// RMSNorm and fused add-bias + residual + RMSNorm for gfx950.
//
// Semantics follow the reference's fp32 kernel (src/kernels/fused_addresidual_norm.cu:55-97):
//   x = out + residual (+ bias);  residual := x;  out := gamma * x * rsqrt(sum(x^2)/H + eps)
// with optional residual and bias.  Design (not the reference's): the whole row stays in fp32
// registers between the sum of squares and the scaling, so every tensor crosses HBM exactly once
// (the reference re-reads and read-modify-writes decoder_out); all global accesses are 16-byte
// vectors; the row sum is a DPP wave reduction plus, when a row spans several waves, one small LDS
// combine behind a single barrier, associated the same way under every launch configuration.
#include <atomic>

#include "norm_rows.h"

namespace isp {

template <typename T, int NV, int WPR, int ST, int BLOCK>
__global__ __launch_bounds__(BLOCK) void fused_norm_rows(T* residual, T* out, const T* bias,
                                                         const T* gamma, float eps, int tokens,
                                                         int hidden, unsigned flags) {
    norm_rows_body<T, NV, WPR, ST, BLOCK, kOpsRuntime>(residual, out, bias, gamma, eps, tokens, hidden, flags);
}

// Any hidden size and any alignment: one workgroup per row, scalar accesses, two passes over the
// inputs (the first only accumulates, the second recomputes x with the same fp32 operations and
// stores), so nothing is overwritten before it has been read for the last time.
template <typename T>
__global__ __launch_bounds__(kBlock) void fused_norm_generic(T* residual, T* out, const T* bias,
                                                             const T* gamma, float eps, int tokens,
                                                             int hidden, unsigned flags) {
    const int row = blockIdx.x;
    T* out_row = out + (size_t)row * hidden;
    T* rsd_row = residual ? residual + (size_t)row * hidden : nullptr;
    float acc = 0.0f;
    for (int i = threadIdx.x; i < hidden; i += kBlock) {
        float x = Elem<T>::to_f32(out_row[i]);
        if (rsd_row) x += Elem<T>::to_f32(rsd_row[i]);
        if (bias) x += Elem<T>::to_f32(bias[i]);
        acc += x * x;
    }
    __shared__ float partial[kBlock / kWave];
    float total = wave_sum(acc);
    if ((threadIdx.x % kWave) == 0) partial[threadIdx.x / kWave] = total;
    __syncthreads();
    total = (partial[0] + partial[1]) + (partial[2] + partial[3]);
    const float inv = rsqrtf(total / (float)hidden + eps);
    for (int i = threadIdx.x; i < hidden; i += kBlock) {
        float x = Elem<T>::to_f32(out_row[i]);
        if (rsd_row) {
            x += Elem<T>::to_f32(rsd_row[i]);
            if (flags & ISP_NORM_RESIDUAL_EXCLUDES_BIAS) rsd_row[i] = Elem<T>::from_f32(x);
        }
        if (bias) x += Elem<T>::to_f32(bias[i]);
        if (rsd_row && !(flags & ISP_NORM_RESIDUAL_EXCLUDES_BIAS)) rsd_row[i] = Elem<T>::from_f32(x);
        out_row[i] = Elem<T>::from_f32(Elem<T>::to_f32(gamma[i]) * x * inv);
    }
}

// ----------------------------------------------------------------------------- launch
constexpr int kMaxWpr = 16;  // 1024 threads
constexpr int kMaxNv = 8;
constexpr int kNvKinds = 4, kWprKinds = 5, kStoreKinds = 3, kBlockKinds = 2;

template <typename T>
using NormKernel = void (*)(T*, T*, const T*, const T*, float, int, int, unsigned);

// One compiled instantiation: the kernel, its workgroup size and the rows a workgroup carries.
template <typename T>
struct NormVariant {
    NormKernel<T> kernel;
    int block, rows_per_block, index;
};

constexpr int log2_of(int v) { return v <= 1 ? 0 : 1 + log2_of(v / 2); }

// BIG selects 512-thread workgroups for rows of up to four waves (two or more rows share a
// workgroup); rows of 8 and 16 waves fill a workgroup on their own.
template <typename T, int NV, int WPR, int ST, bool BIG>
static NormVariant<T> variant_of() {
    constexpr int MIN = norm_block(WPR);
    constexpr int BLOCK = (BIG && MIN < 512) ? 512 : MIN;
    constexpr int index = ((log2_of(NV) * kWprKinds + log2_of(WPR)) * kStoreKinds + ST) * kBlockKinds + (BIG ? 1 : 0);
    return {fused_norm_rows<T, NV, WPR, ST, BLOCK>, BLOCK, BLOCK / (kWave * WPR), index};
}

template <typename T, int NV, int WPR>
static NormVariant<T> variant_st(int st, bool big) {
    if (st == kStoreThrough) return big ? variant_of<T, NV, WPR, kStoreThrough, true>() : variant_of<T, NV, WPR, kStoreThrough, false>();
    if (st == kStoreStream) return big ? variant_of<T, NV, WPR, kStoreStream, true>() : variant_of<T, NV, WPR, kStoreStream, false>();
    return big ? variant_of<T, NV, WPR, kStorePlain, true>() : variant_of<T, NV, WPR, kStorePlain, false>();
}

template <typename T, int WPR>
static NormVariant<T> variant_nv(int nv, int st, bool big) {
    if (nv <= 1) return variant_st<T, 1, WPR>(st, big);
    if (nv <= 2) return variant_st<T, 2, WPR>(st, big);
    if (nv <= 4) return variant_st<T, 4, WPR>(st, big);
    return variant_st<T, 8, WPR>(st, big);
}

// wpr in {1, 2, 4, 8, 16}; nv = vectors per lane (rounded up to 1, 2, 4 or 8 here).
template <typename T>
static NormVariant<T> norm_variant(int wpr, int nv, int st, bool big) {
    switch (wpr) {
        case 1: return variant_nv<T, 1>(nv, st, big);
        case 2: return variant_nv<T, 2>(nv, st, big);
        case 4: return variant_nv<T, 4>(nv, st, big);
        case 8: return variant_nv<T, 8>(nv, st, big);
        default: return variant_nv<T, 16>(nv, st, big);
    }
}

// Token rows one launch of this instantiation keeps resident on the device at once: workgroups per
// compute unit as the runtime's occupancy calculator reports them for the compiled kernel (its
// register and LDS use decide), times compute units, times rows per workgroup.  Asked once per
// instantiation and process; every device of one process is assumed to be the same gfx950 part.
template <typename T>
static long long resident_rows(const NormVariant<T>& v) {
    static std::atomic<int> blocks_per_cu[kNvKinds * kWprKinds * kStoreKinds * kBlockKinds] = {};
    int n = blocks_per_cu[v.index].load(std::memory_order_relaxed);
    if (n == 0) {
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, reinterpret_cast<const void*>(v.kernel), v.block, 0) !=
                hipSuccess || n <= 0) {
            (void)hipGetLastError();
            n = (kWave * 32) / v.block;  // 8 wavefronts per SIMD
            if (n < 1) n = 1;
        }
        blocks_per_cu[v.index].store(n, std::memory_order_relaxed);
    }
    return (long long)n * (resident_waves() / 32) * v.rows_per_block;
}

struct NormPlan {
    int wpr, nv, store, block_big;
    bool streaming;  // kNormStreamingOrder
    bool few;        // every wave of the launch is resident at once: fused_norm_few_rows if it is compiled for the shape
    bool pacing;     // kNormPacingLoad
};

// Operand combination of a call as the few-rows kernels know them, or kOpsRuntime if they do not.
inline int few_rows_ops(bool has_res, bool has_bias, unsigned flags) {
    if (flags & ISP_NORM_RESIDUAL_EXCLUDES_BIAS) return kOpsRuntime;
    if (!has_res) return has_bias ? kOpsRuntime : kOpsNone;
    return has_bias ? kOpsResidualBias : kOpsResidual;
}

// The launch configuration for `tokens` rows of `nvec` 16-byte vectors.
template <typename T>
static NormPlan plan_norm(int tokens, int nvec, bool fused, bool has_bias = true) {
    auto vectors_per_lane = [nvec](int w) { return (nvec + kWave * w - 1) / (kWave * w); };
    // in place on both tensors: plain non-temporal stores measured best (write-through costs 2 %) -- except
    // where a launch writes no more than 1 MiB: ordinary stores, which the L2 acknowledges, then end the
    // kernel sooner (16 x 4096 fp32: 2.13 against 2.56 us per launch; equal at 1 MiB; 2 % slower at 2 MiB)
    const size_t written = (size_t)tokens * (size_t)nvec * 16u * (fused ? 2u : 1u);
    const int kind = store_kind(tuning(ISP_TUNE_NORM_STORE), written <= (1u << 20) ? kStorePlain : kStoreStream);
    const int block_knob = tuning(ISP_TUNE_NORM_BLOCK_THREADS);
    int wpr = tuning(ISP_TUNE_NORM_WAVES_PER_ROW);
    if (wpr != 1 && wpr != 2 && wpr != 4 && wpr != 8 && wpr != 16) {
        // Automatic, from sweeps over 256..16384 rows of 4096 elements, both types:
        //  * streaming regime (several rounds of waves): about two 16-byte loads in flight
        //    per lane, i.e. waves per row = vectors x operand streams / 128, rounded to the
        //    nearest power of two;
        //  * if that needs more rows resident than the device holds at once, but fewer waves per
        //    row fit the whole launch into a single round, take the single round: every load is
        //    then issued at kernel start (5-10 % faster).  Whether a configuration fits is asked
        //    of the occupancy calculator, because more vectors per lane mean more registers and
        //    fewer resident waves (2 vectors per lane: 8 waves per SIMD, 4: 7, 8: 4);
        //  * with a residual operand, a single round that is at least twice as large as it needs
        //    to be to occupy half the machine: half the waves per row (two vectors of each
        //    operand in flight per lane) measured 5 % faster;
        //  * few rows: split rows further, down to one vector per lane, to occupy the machine.
        const int streams = fused ? 2 : 1;
        const int want = nvec * streams;  // 16-byte loads per row
        wpr = 1;
        while (wpr < kMaxWpr && 3 * kWave * wpr < want) wpr *= 2;  // 2^round(log2(want / 128))
        while (wpr < kMaxWpr && vectors_per_lane(wpr) > kMaxNv) wpr *= 2;
        auto fits = [&](int w) {
            return vectors_per_lane(w) <= kMaxNv &&
                   (long long)tokens <= resident_rows(norm_variant<T>(w, vectors_per_lane(w), kind, false));
        };
        if (!fits(wpr)) {
            for (int w = wpr / 2; w >= 1 && vectors_per_lane(w) <= kMaxNv; w /= 2) {
                if (fits(w)) {
                    wpr = w;
                    break;
                }
            }
        } else {
            const long long half = resident_waves() / 2;
            while (wpr < kMaxWpr && vectors_per_lane(wpr) > 1 && (long long)tokens * wpr < half) wpr *= 2;
            while (fused && wpr > 1 && (long long)tokens * (wpr / 2) >= half &&
                   vectors_per_lane(wpr / 2) <= 2 && fits(wpr / 2))
                wpr /= 2;
        }
        // A plain RMSNorm launch whose rows, split down to one vector per lane, are all resident at once takes
        // that split: it is the one the kernels with the operand set fixed at compile time are built for (1024 x
        // 4096 fp16: 3.98 against 4.60 us; 512 x 4096 fp32: 3.98 against 4.36).  With a residual the two splits
        // are within 3 % of each other either way at that size, and the rule above stands.
        if (!fused) {
            int one = 1;
            while (one < kMaxWpr && vectors_per_lane(one) > 1) one *= 2;
            if (vectors_per_lane(one) == 1 && (long long)tokens * one <= (long long)resident_waves()) wpr = one;
        }
    }
    while (wpr < kMaxWpr && vectors_per_lane(wpr) > kMaxNv) wpr *= 2;
    // 512-thread workgroups (two or four rows each) for 16-bit rows of two or four waves: half as
    // many workgroups for the dispatcher to place before the last row's loads are out (+1 % at
    // 2048 x 4096 with a residual, 0.5-3 % elsewhere; with 32-bit elements, and with one wave per
    // row, the 256-thread workgroup measured 1-6 % faster)
    const bool big = block_knob >= 512 || (block_knob <= 0 && (wpr == 4 || wpr == 2) && sizeof(T) == 2);
    const int order = tuning(ISP_TUNE_NORM_ORDER);
    const bool streaming = order == 2;
    // see kNormPacingLoad; knob values 4 / 5 switch it off / on for every residual-without-bias launch
    const bool one_round = (long long)tokens <= resident_rows(norm_variant<T>(wpr, vectors_per_lane(wpr), kind, big));
    const size_t read_bytes = (size_t)tokens * (size_t)nvec * 16u * 2u;
    const bool pacing = fused && !has_bias && !streaming && order != 4 &&
                        (order == 5 || (one_round && read_bytes > (24u << 20)));
    // The kernels with the operand set fixed at compile time (and their arguments preloaded) take every launch
    // whose waves are all resident at once, as far as they are compiled (one vector per lane; two with 16 waves
    // per row) -- measured 5-13 % faster than the general kernel up to there (768 x 4096 fp16: 5.1 against 5.5 us
    // with a residual, 3.55 against 3.98 without), except where the launch wants the pacing load, which only the
    // general kernel has (1024 x 4096 fp32 with a residual and no bias: 12.9 against 11.1 us).
    const bool few = !streaming && !pacing && order != 3 && (long long)tokens * wpr <= (long long)resident_waves();
    return {wpr, vectors_per_lane(wpr), kind, big ? 1 : 0, streaming, few, pacing};
}

template <typename T>
static int fused_norm(void* residual_, void* out_, const void* bias_, const void* gamma_, float eps,
                      int tokens, int hidden, unsigned flags, hipStream_t s) {
    if (tokens < 0 || hidden < 0) return ISP_ERR_BAD_SHAPE;
    if (tokens == 0 || hidden == 0) return ISP_OK;
    ISP_REQUIRE_PTR(out_);
    ISP_REQUIRE_PTR(gamma_);
    T* residual = static_cast<T*>(residual_);
    T* out = static_cast<T*>(out_);
    const T* bias = static_cast<const T*>(bias_);
    const T* gamma = static_cast<const T*>(gamma_);
    constexpr int VEC = Elem<T>::kVec;

    const bool vec_ok = (hidden % VEC == 0) && aligned16(out) && aligned16(gamma) &&
                        (!residual || aligned16(residual)) && (!bias || aligned16(bias)) &&
                        (hidden / VEC) <= kMaxNv * kWave * kMaxWpr;
    if (!vec_ok) {
        hipLaunchKernelGGL((fused_norm_generic<T>), dim3((unsigned)tokens), dim3(kBlock), 0, s,
                           residual, out, bias, gamma, eps, tokens, hidden, flags & ~kNormInternalFlags);
    } else {
        const NormPlan plan = plan_norm<T>(tokens, hidden / VEC, residual != nullptr, bias != nullptr);
        const int ops = few_rows_ops(residual != nullptr, bias != nullptr, flags);
        const NormFewKernel<T> few =
            plan.few && ops != kOpsRuntime ? norm_few_variant<T>(plan.wpr, plan.nv, plan.store, ops) : nullptr;
        if (few != nullptr) {
            const int block = norm_block(plan.wpr), rows_per_block = block / (kWave * plan.wpr);
            hipLaunchKernelGGL(few, dim3((unsigned)((tokens + rows_per_block - 1) / rows_per_block)), dim3(block), 0,
                               s, residual, out, bias, gamma, eps, tokens, hidden);
        } else {
            const NormVariant<T> v = norm_variant<T>(plan.wpr, plan.nv, plan.store, plan.block_big != 0);
            const dim3 grid((unsigned)((tokens + v.rows_per_block - 1) / v.rows_per_block));
            hipLaunchKernelGGL(v.kernel, grid, dim3(v.block), 0, s, residual, out, bias, gamma, eps, tokens, hidden,
                               (flags & ~kNormInternalFlags) | (plan.streaming ? kNormStreamingOrder : 0u) |
                                   (plan.pacing ? kNormPacingLoad : 0u));
        }
    }
    return note_launch(hipGetLastError());
}

template <typename T>
static int describe_plan(int tokens, int hidden, int fused, int* wpr, int* nv, int* block, int* store) {
    constexpr int VEC = Elem<T>::kVec;
    if (tokens <= 0 || hidden <= 0) return ISP_ERR_BAD_SHAPE;
    if (hidden % VEC != 0 || hidden / VEC > kMaxNv * kWave * kMaxWpr) return ISP_ERR_UNSUPPORTED;
    const NormPlan plan = plan_norm<T>(tokens, hidden / VEC, fused != 0);
    const NormVariant<T> v = norm_variant<T>(plan.wpr, plan.nv, plan.store, plan.block_big != 0);
    if (wpr) *wpr = plan.wpr;
    if (nv) *nv = plan.nv <= 1 ? 1 : plan.nv <= 2 ? 2 : plan.nv <= 4 ? 4 : 8;
    if (block) *block = v.block;
    if (store) *store = plan.store;
    return ISP_OK;
}

// 1 if a call with these operands takes a few-rows kernel, 0 if the general one, < 0 if neither applies.
template <typename T>
static int describe_variant(int tokens, int hidden, int has_residual, int has_bias, unsigned flags) {
    constexpr int VEC = Elem<T>::kVec;
    if (tokens <= 0 || hidden <= 0) return ISP_ERR_BAD_SHAPE;
    if (hidden % VEC != 0 || hidden / VEC > kMaxNv * kWave * kMaxWpr) return ISP_ERR_UNSUPPORTED;
    const NormPlan plan = plan_norm<T>(tokens, hidden / VEC, has_residual != 0, has_bias != 0);
    const int ops = few_rows_ops(has_residual != 0, has_bias != 0, flags);
    return plan.few && ops != kOpsRuntime && norm_few_variant<T>(plan.wpr, plan.nv, plan.store, ops) != nullptr ? 1 : 0;
}

}  // namespace isp

extern "C" {

int isp_norm_launch_variant(int elem_size, int tokens, int hidden, int has_residual, int has_bias, unsigned flags) {
    if (elem_size == 2) return isp::describe_variant<__half>(tokens, hidden, has_residual, has_bias, flags);
    if (elem_size == 4) return isp::describe_variant<float>(tokens, hidden, has_residual, has_bias, flags);
    return ISP_ERR_BAD_SHAPE;
}

int isp_norm_launch_config(int elem_size, int tokens, int hidden, int fused, int* waves_per_row,
                           int* vectors_per_lane, int* block_threads, int* store_kind) {
    if (elem_size == 2)
        return isp::describe_plan<__half>(tokens, hidden, fused, waves_per_row, vectors_per_lane, block_threads, store_kind);
    if (elem_size == 4)
        return isp::describe_plan<float>(tokens, hidden, fused, waves_per_row, vectors_per_lane, block_threads, store_kind);
    return ISP_ERR_BAD_SHAPE;
}

int isp_fused_add_bias_residual_rmsnorm_f32(void* residual, void* decoder_out, const void* bias,
                                            const void* gamma, float eps, int tokens, int hidden,
                                            unsigned flags, isp_stream_t stream) {
    return isp::fused_norm<float>(residual, decoder_out, bias, gamma, eps, tokens, hidden, flags,
                                  static_cast<hipStream_t>(stream));
}

int isp_fused_add_bias_residual_rmsnorm_f16(void* residual, void* decoder_out, const void* bias,
                                            const void* gamma, float eps, int tokens, int hidden,
                                            unsigned flags, isp_stream_t stream) {
    return isp::fused_norm<__half>(residual, decoder_out, bias, gamma, eps, tokens, hidden, flags,
                                   static_cast<hipStream_t>(stream));
}

int isp_rmsnorm_f32(void* x, const void* gamma, float eps, int tokens, int hidden,
                    isp_stream_t stream) {
    return isp::fused_norm<float>(nullptr, x, nullptr, gamma, eps, tokens, hidden, 0u,
                                  static_cast<hipStream_t>(stream));
}

int isp_rmsnorm_f16(void* x, const void* gamma, float eps, int tokens, int hidden,
                    isp_stream_t stream) {
    return isp::fused_norm<__half>(nullptr, x, nullptr, gamma, eps, tokens, hidden, 0u,
                                   static_cast<hipStream_t>(stream));
}

}  // extern "C"
