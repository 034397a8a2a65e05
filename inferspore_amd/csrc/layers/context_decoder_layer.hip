// LlamaContextDecoderLayer: one LLaMA prefill layer over the reference's data model (see the header
// for the sequence).  This file holds the parts that are not this library's launch* kernels: the
// hipBLASLt GEMM calls (shape cases of the reference's src/kernels/linear.cu:7-15, 67-109) and a plain
// masked softmax for the attention scores.
#include "src/layers/decoder/context_decoder_layer.h"

#include <hipblaslt/hipblaslt.h>
#include <hipblaslt/hipblaslt-ext.hpp>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <tuple>
#include <type_traits>
#include <utility>
#include <vector>
#include <algorithm>

#include "src/kernels/act_kernel.h"
#include "src/kernels/fused_addresidual_norm.h"
#include "src/kernels/fused_transpose_and_remv_pad.h"
#include "src/kernels/qkv_bias_and_RoPE.h"
#include "src/kernels/repeat_kv.h"
#include "src/utils/macro.h"

namespace isp_layers {

#define ISP_LT_CHECK(call)                                                                          \
    do {                                                                                            \
        const hipblasStatus_t isp_lt_status_ = (call);                                              \
        LLM_CHECK_WITH_INFO(isp_lt_status_ == HIPBLAS_STATUS_SUCCESS,                               \
                            std::string("hipBLASLt call failed with status ") +                     \
                                std::to_string((int)isp_lt_status_) + ": " #call);                  \
    } while (0)

template <typename T>
struct LtType;
template <>
struct LtType<float> {
    static constexpr hipDataType value = HIP_R_32F;
};
template <>
struct LtType<half> {
    static constexpr hipDataType value = HIP_R_16F;
};

// Row-major C[m, n] = alpha * A[m, k] x op(W), fp32 accumulation, optionally strided-batched.
//   w_is_nk:  W is stored [n, k] (a weight kept [out_features, in_features], or the keys of
//             q x k^T), else [k, n].
// hipBLASLt is column-major, so the call computes C^T = op(W)^T x A^T: its "A" operand is W, its
// "B" operand is the activation, and a row-major [r, c] matrix is a column-major [c, r] one.
//
// The algorithm of a shape is chosen when the shape is first seen.  The library's heuristic proposes up to 16
// (ISP_LAYERS_GEMM_CANDIDATES changes the number, up to 4096), and unless ISP_LAYERS_GEMM_AUTOTUNE=0 each is run on the
// call's own operands (beta is 0 and no output aliases an input, so repeating the product is harmless) and the
// fastest is kept -- the first proposal is not always the fastest on a given device.  That measurement is bounded:
// it is made once per BUCKET of shapes (the row count rounded up to a multiple of 256, or to a power of two below
// that; for the batched attention products also n and k rounded up to multiples of 64), so the ragged token counts
// of successive prompt batches share one measurement -- a shape whose bucket has been measured takes the bucket's
// algorithm after asking the library that it supports the exact shape -- and at most kMaxTuned buckets are ever
// measured; later ones take the heuristic's first proposal.  The per-shape descriptor cache is emptied when it
// reaches kMaxPlans entries.  ISP_LAYERS_GEMM_VERBOSE=1 prints each choice.
class GemmEngine {
public:
    explicit GemmEngine(BaseAllocator* allocator) : allocator_(allocator) {
        const char* env = std::getenv("ISP_LAYERS_GEMM_AUTOTUNE");
        autotune_ = !(env != nullptr && std::strcmp(env, "0") == 0);
        const char* many = std::getenv("ISP_LAYERS_GEMM_CANDIDATES");
        if (many != nullptr && std::atoi(many) > 0) candidates_ = std::min(std::atoi(many), kMaxCandidates);
        ISP_LT_CHECK(hipblasLtCreate(&handle_));
        workspace_ = allocator_->UnifyMalloc(nullptr, kWorkspaceBytes, false);
        ISP_LT_CHECK(hipblasLtMatmulPreferenceCreate(&pref_));
        const uint64_t ws = kWorkspaceBytes;
        ISP_LT_CHECK(hipblasLtMatmulPreferenceSetAttribute(pref_, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws,
                                                           sizeof(ws)));
    }
    ~GemmEngine() {
        for (auto& kv : plans_) destroy(kv.second);
        if (pref_) (void)hipblasLtMatmulPreferenceDestroy(pref_);
        if (workspace_) allocator_->UnifyFree(workspace_, false);
        if (handle_) (void)hipblasLtDestroy(handle_);
    }
    GemmEngine(const GemmEngine&) = delete;
    GemmEngine& operator=(const GemmEngine&) = delete;

    void matmul(hipDataType type, const void* a, const void* w, void* c, int m, int n, int k, bool w_is_nk,
                int lda, int ldw, int ldc, int batch = 1, long long stride_a = 0, long long stride_w = 0,
                long long stride_c = 0, float alpha = 1.0f) {
        if (m == 0 || n == 0 || batch == 0) return;
        const Key key{(int)type, m, n, k, w_is_nk ? 1 : 0, lda, ldw, ldc, batch, stride_a, stride_w, stride_c};
        auto it = plans_.find(key);
        if (it == plans_.end()) {
            if (plans_.size() >= kMaxPlans) {
                for (auto& kv : plans_) destroy(kv.second);
                plans_.clear();
            }
            it = plans_.emplace(key, plan(type, key, a, w, c, alpha)).first;
        }
        const Plan& p = it->second;
        const float beta = 0.0f;
        ISP_LT_CHECK(hipblasLtMatmul(handle_, p.desc, &alpha, w, p.w, a, p.a, &beta, c, p.c, c, p.c, &p.algo,
                                     workspace_, kWorkspaceBytes, nullptr));
    }

private:
    static constexpr size_t kWorkspaceBytes = 32u << 20;
    static constexpr int kMaxCandidates = 4096;
    static constexpr size_t kMaxTuned = 64;    // buckets of shapes whose algorithm is measured
    static constexpr size_t kMaxPlans = 1024;  // exact shapes whose descriptors are kept
    using Key = std::tuple<int, int, int, int, int, int, int, int, int, long long, long long, long long>;
    struct Plan {
        hipblasLtMatmulDesc_t desc = nullptr;
        hipblasLtMatrixLayout_t w = nullptr, a = nullptr, c = nullptr;
        hipblasLtMatmulAlgo_t algo;
    };

    static int bucket_rows(int v) {
        if (v > 256) return (v + 255) / 256 * 256;
        int p = 1;
        while (p < v) p *= 2;
        return p;
    }
    // The shape a measurement is shared by: rows rounded up; for batched products (the padded attention, whose n, k,
    // leading dimensions and strides all follow the batch's longest query and context) those rounded or dropped too.
    static Key bucket_of(const Key& key) {
        int m, n, k, nk, lda, ldw, ldc, batch, t;
        long long sa, sw, sc;
        std::tie(t, m, n, k, nk, lda, ldw, ldc, batch, sa, sw, sc) = key;
        if (batch > 1) return Key{t, bucket_rows(m), (n + 63) / 64 * 64, (k + 63) / 64 * 64, nk, 0, 0, 0, batch, 0, 0, 0};
        return Key{t, bucket_rows(m), n, k, nk, lda, ldw, ldc, batch, sa, sw, sc};
    }

    static void batched(hipblasLtMatrixLayout_t layout, int batch, long long stride) {
        if (batch <= 1) return;
        const int32_t count = batch;
        const int64_t offset = stride;
        ISP_LT_CHECK(hipblasLtMatrixLayoutSetAttribute(layout, HIPBLASLT_MATRIX_LAYOUT_BATCH_COUNT, &count, sizeof(count)));
        ISP_LT_CHECK(hipblasLtMatrixLayoutSetAttribute(layout, HIPBLASLT_MATRIX_LAYOUT_STRIDED_BATCH_OFFSET, &offset,
                                                       sizeof(offset)));
    }

    // Milliseconds per product with `algo` (two untimed runs, then the mean of `runs`); negative if it fails.
    float time_algo(const Plan& p, const hipblasLtMatmulAlgo_t& algo, const void* a, const void* w, void* c,
                    float alpha, int runs = 5) {
        const float beta = 0.0f;
        hipEvent_t e0, e1;
        if (hipEventCreate(&e0) != hipSuccess) return -1.0f;
        if (hipEventCreate(&e1) != hipSuccess) {
            (void)hipEventDestroy(e0);
            return -1.0f;
        }
        float ms = -1.0f;
        bool ok = true;
        for (int i = 0; i < 2 + runs && ok; i++) {
            if (i == 2) ok = hipEventRecord(e0, nullptr) == hipSuccess;
            ok = ok && hipblasLtMatmul(handle_, p.desc, &alpha, w, p.w, a, p.a, &beta, c, p.c, c, p.c, &algo,
                                       workspace_, kWorkspaceBytes, nullptr) == HIPBLAS_STATUS_SUCCESS;
        }
        if (ok && hipEventRecord(e1, nullptr) == hipSuccess && hipEventSynchronize(e1) == hipSuccess &&
            hipEventElapsedTime(&ms, e0, e1) == hipSuccess)
            ms /= (float)runs;
        else
            ms = -1.0f;
        (void)hipGetLastError();
        (void)hipEventDestroy(e0);
        (void)hipEventDestroy(e1);
        return ms;
    }

    Plan plan(hipDataType type, const Key& key, const void* a, const void* w, void* c, float alpha) {
        int m, n, k, nk, lda, ldw, ldc, batch, t;
        long long sa, sw, sc;
        std::tie(t, m, n, k, nk, lda, ldw, ldc, batch, sa, sw, sc) = key;
        Plan p;
        ISP_LT_CHECK(hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F));
        const hipblasOperation_t op_w = nk ? HIPBLAS_OP_T : HIPBLAS_OP_N, op_a = HIPBLAS_OP_N;
        ISP_LT_CHECK(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_w, sizeof(op_w)));
        ISP_LT_CHECK(hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_a, sizeof(op_a)));
        // column-major views: W [n, k] row-major = [k, n] column-major (transposed by op_w);
        // W [k, n] row-major = [n, k] column-major; A [m, k] row-major = [k, m]; C [m, n] = [n, m]
        if (nk) ISP_LT_CHECK(hipblasLtMatrixLayoutCreate(&p.w, type, (uint64_t)k, (uint64_t)n, ldw));
        else ISP_LT_CHECK(hipblasLtMatrixLayoutCreate(&p.w, type, (uint64_t)n, (uint64_t)k, ldw));
        ISP_LT_CHECK(hipblasLtMatrixLayoutCreate(&p.a, type, (uint64_t)k, (uint64_t)m, lda));
        ISP_LT_CHECK(hipblasLtMatrixLayoutCreate(&p.c, type, (uint64_t)n, (uint64_t)m, ldc));
        batched(p.w, batch, sw);
        batched(p.a, batch, sa);
        batched(p.c, batch, sc);
        std::vector<hipblasLtMatmulHeuristicResult_t> found(candidates_);
        int count = 0;
        ISP_LT_CHECK(hipblasLtMatmulAlgoGetHeuristic(handle_, p.desc, p.w, p.a, p.c, p.c, pref_,
                                                     autotune_ ? candidates_ : 1, found.data(), &count));
        LLM_CHECK_WITH_INFO(count > 0, "hipBLASLt offers no algorithm for a GEMM of this layer");
        int best = 0;
        float best_ms = -1.0f;
        const char* how = "the heuristic's first proposal";
        const Key tuned_key = bucket_of(key);
        auto known = tuned_.find(tuned_key);
        if (autotune_ && known != tuned_.end()) {
            // the bucket's measured algorithm, if the library runs it on this exact shape within the workspace
            const float beta = 0.0f;
            size_t need = 0;
            hipblasLtMatmulAlgo_t algo = known->second;
            if (hipblaslt_ext::matmulIsAlgoSupported(handle_, p.desc, &alpha, p.w, p.a, &beta, p.c, p.c, algo, need) ==
                    HIPBLAS_STATUS_SUCCESS && need <= kWorkspaceBytes) {
                p.algo = algo;
                if (std::getenv("ISP_LAYERS_GEMM_VERBOSE") != nullptr)
                    std::fprintf(stderr, "[isp_layers] GEMM m=%d n=%d k=%d batch=%d: the algorithm measured for its bucket\n", m, n, k, batch);
                return p;
            }
        } else if (autotune_ && count > 1 && tuned_.size() < kMaxTuned) {
            how = "measured";
            // a first pass over every proposal, then the four fastest again over more runs: differences of a
            // per cent or two between the leaders are inside the noise of five runs
            std::vector<std::pair<float, int>> timed;
            for (int i = 0; i < count; i++) {
                if (found[i].workspaceSize > kWorkspaceBytes) continue;
                const float ms = time_algo(p, found[i].algo, a, w, c, alpha);
                if (ms >= 0.0f) timed.emplace_back(ms, i);
            }
            std::sort(timed.begin(), timed.end());
            for (size_t j = 0; j < timed.size() && j < 4; j++) {
                const float ms = timed.size() > 1 ? time_algo(p, found[timed[j].second].algo, a, w, c, alpha, 20) : timed[j].first;
                if (ms >= 0.0f && (best_ms < 0.0f || ms < best_ms)) {
                    best_ms = ms;
                    best = timed[j].second;
                }
            }
            tuned_.emplace(tuned_key, found[best].algo);
        }
        if (std::getenv("ISP_LAYERS_GEMM_VERBOSE") != nullptr)
            std::fprintf(stderr, "[isp_layers] GEMM m=%d n=%d k=%d batch=%d: proposal %d of %d (%s)%s\n", m, n, k, batch, best,
                         count, how, best_ms >= 0.0f ? (", " + std::to_string(best_ms * 1e3f) + " us").c_str() : "");
        p.algo = found[best].algo;
        return p;
    }

    static void destroy(Plan& p) {
        if (p.w) (void)hipblasLtMatrixLayoutDestroy(p.w);
        if (p.a) (void)hipblasLtMatrixLayoutDestroy(p.a);
        if (p.c) (void)hipblasLtMatrixLayoutDestroy(p.c);
        if (p.desc) (void)hipblasLtMatmulDescDestroy(p.desc);
    }

    BaseAllocator* allocator_;
    hipblasLtHandle_t handle_ = nullptr;
    hipblasLtMatmulPreference_t pref_ = nullptr;
    void* workspace_ = nullptr;
    bool autotune_ = true;
    int candidates_ = 16;
    std::map<Key, Plan> plans_;                     // exact shapes: descriptors and the algorithm in use
    std::map<Key, hipblasLtMatmulAlgo_t> tuned_;    // buckets of shapes: the algorithm that measured fastest
};

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(half x) { return __half2float(x); }
__device__ __forceinline__ void from_float(float x, float* p) { *p = x; }
__device__ __forceinline__ void from_float(float x, half* p) { *p = __float2half_rn(x); }

__device__ __forceinline__ float block_reduce(float v, bool take_max, float* shared) {
    for (int off = 32; off > 0; off >>= 1) {
        const float o = __shfl_xor(v, off, 64);
        v = take_max ? fmaxf(v, o) : v + o;
    }
    const int wave = threadIdx.x / 64, waves = blockDim.x / 64;
    __syncthreads();  // `shared` may still be read from the previous reduction
    if ((threadIdx.x % 64) == 0) shared[wave] = v;
    __syncthreads();
    v = shared[0];
    for (int w = 1; w < waves; w++) v = take_max ? fmaxf(v, shared[w]) : v + shared[w];
    return v;
}

// In place on scores [batch, head_num, max_q_len, max_k_len]: row (b, h, q) becomes
// softmax(scale * scores) over the keys query q may see -- key positions <= history_length[b] + q and
// < context_length[b] -- and zero elsewhere; rows of padded queries (q >= input_length[b]) become zero.
// What the reference does with launchBuildCausalMasks + launchScaleMaskAndSoftmax
// (src/kernels/build_casual_mask.cu:5-42, attn_softmax_kernel.cu:50-125), with the mask computed
// from the lengths instead of read from a [batch, q, k] tensor -- and with the history keys visible,
// which the reference's mask hides (build_casual_mask.cu:36: k >= klen - qlen; see the header).
// fp32 arithmetic.
template <typename T>
__global__ __launch_bounds__(256) void masked_scaled_softmax(T* scores, const int* history_length,
                                                             const int* input_length,
                                                             const int* context_length, int head_num,
                                                             int max_q_len, int max_k_len, float scale) {
    __shared__ float shared[4];
    const int q = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    T* row = scores + (((size_t)b * head_num + h) * max_q_len + q) * (size_t)max_k_len;
    int visible = 0;
    if (q < input_length[b]) {
        visible = history_length[b] + q + 1;
        if (visible > context_length[b]) visible = context_length[b];
        if (visible > max_k_len) visible = max_k_len;
    }
    float m = -INFINITY;
    for (int i = threadIdx.x; i < visible; i += blockDim.x) m = fmaxf(m, scale * to_float(row[i]));
    m = block_reduce(m, true, shared);
    float sum = 0.0f;
    for (int i = threadIdx.x; i < visible; i += blockDim.x) sum += expf(scale * to_float(row[i]) - m);
    sum = block_reduce(sum, false, shared);
    const float inv = visible > 0 ? 1.0f / sum : 0.0f;
    for (int i = threadIdx.x; i < max_k_len; i += blockDim.x) {
        const float p = i < visible ? expf(scale * to_float(row[i]) - m) * inv : 0.0f;
        from_float(p, row + i);
    }
}

// Lane exchange inside the VALU (no LDS traffic); `ctrl` is the DPP control word.
template <int ctrl>
__device__ __forceinline__ float lane_swap(float x) {
    return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), ctrl, 0xf, 0xf, true));
}
__device__ __forceinline__ float read_lane(float x, int lane) {
    return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(x), lane));
}
// Maximum / sum over the 64 lanes, the result in every lane: quad swaps and the two row mirrors fold each
// row of 16 lanes, the four row results are combined as scalars.
__device__ __forceinline__ float wave_max(float x) {
    x = fmaxf(x, lane_swap<0xB1>(x));
    x = fmaxf(x, lane_swap<0x4E>(x));
    x = fmaxf(x, lane_swap<0x141>(x));
    x = fmaxf(x, lane_swap<0x140>(x));
    return fmaxf(fmaxf(read_lane(x, 0), read_lane(x, 16)), fmaxf(read_lane(x, 32), read_lane(x, 48)));
}
__device__ __forceinline__ float wave_total(float x) {
    x += lane_swap<0xB1>(x);
    x += lane_swap<0x4E>(x);
    x += lane_swap<0x141>(x);
    x += lane_swap<0x140>(x);
    return (read_lane(x, 0) + read_lane(x, 16)) + (read_lane(x, 32) + read_lane(x, 48));
}
__device__ __forceinline__ int uniform_i32(const int* p, int i) {
    // the lengths never change while a kernel runs: read them through the scalar cache
    typedef const int __attribute__((address_space(4)))* constant_ints;
    return reinterpret_cast<constant_ints>((unsigned long long)p)[i];
}

// The same, one wavefront per row with the row in registers: NVW 16-byte vectors per lane cover rows of
// up to 64 * NVW vectors (512 * NVW fp16 keys), every element is read once and written once, vectors that
// lie wholly behind the visible keys are not read at all, and rows of padded queries are only zeroed.
// The kernel is bound as much by its instruction count as by memory (a 1 KiB row per wavefront), so the
// grid's three dimensions name (query / 4, head, batch) and no index is divided, the reductions stay in
// the VALU, the scale is folded into the exponent -- p = 2^(x * c - max(x) * c) with c = scale * log2(e),
// the maximum taken over the raw scores since scale > 0 -- and masked keys are set to -inf once, which the
// hardware exponential turns into exactly 0.  That exponential has a relative error of about 2^-22, far
// inside what the attention output is compared at.  Used when max_k_len is a whole number of vectors and
// fits; else the kernel above.
template <typename T, int NVW>
__global__ __launch_bounds__(256) void masked_scaled_softmax_rows(T* scores, const int* history_length,
                                                                  const int* input_length,
                                                                  const int* context_length, int max_q_len,
                                                                  int max_k_len, float scale_log2e) {
    constexpr int VEC = 16 / (int)sizeof(T);
    union Vec16 {
        uint4 raw;
        T e[VEC];
    };
    const int lane = threadIdx.x % 64;
    const int q = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * 4 + threadIdx.x / 64));
    if (q >= max_q_len) return;  // wave-uniform
    const int b = blockIdx.z;
    int visible = 0;
    if (q < uniform_i32(input_length, b)) {
        visible = min(min(uniform_i32(history_length, b) + q + 1, uniform_i32(context_length, b)), max_k_len);
    }
    T* row = scores + (((size_t)b * gridDim.y + blockIdx.y) * (size_t)max_q_len + (size_t)q) * (size_t)max_k_len;
    const int nvec = max_k_len / VEC;
    if (visible <= 0) {  // wave-uniform: a padded query
#pragma unroll
        for (int j = 0; j < NVW; j++) {
            const int vi = lane + 64 * j;
            if (vi < nvec) *reinterpret_cast<uint4*>(row + vi * VEC) = make_uint4(0u, 0u, 0u, 0u);
        }
        return;
    }
    float x[NVW][VEC];
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < NVW; j++) {
        const int k0 = (lane + 64 * j) * VEC;
        const int left = visible - k0;  // keys of this vector that are visible, if positive (visible <= max_k_len)
        Vec16 v;
        v.raw = make_uint4(0u, 0u, 0u, 0u);
        if (left > 0) v.raw = *reinterpret_cast<const uint4*>(row + k0);
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            x[j][e] = e < left ? to_float(v.e[e]) : -INFINITY;
            m = fmaxf(m, x[j][e]);
        }
    }
    m = wave_max(m);
    const float mc = m * scale_log2e;
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < NVW; j++) {
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            x[j][e] = __builtin_amdgcn_exp2f(fmaf(x[j][e], scale_log2e, -mc));
            sum += x[j][e];
        }
    }
    sum = wave_total(sum);
    const float inv = 1.0f / sum;  // at least 2^0 went into the sum
#pragma unroll
    for (int j = 0; j < NVW; j++) {
        const int vi = lane + 64 * j;
        if (vi < nvec) {
            Vec16 v;
#pragma unroll
            for (int e = 0; e < VEC; e++) from_float(x[j][e] * inv, &v.e[e]);
            *reinterpret_cast<uint4*>(row + vi * VEC) = v.raw;
        }
    }
}

template <typename T>
void launch_masked_scaled_softmax(T* scores, const int* history_length, const int* input_length,
                                  const int* context_length, int batch, int head_num, int max_q_len,
                                  int max_k_len, float scale) {
    constexpr int VEC = 16 / (int)sizeof(T);
    const int nvec = max_k_len / VEC;
    LLM_CHECK_WITH_INFO(batch > 0 && head_num > 0 && max_q_len > 0 && max_k_len > 0 && batch <= 65535 && head_num <= 65535,
                        "attention scores of an extent no grid holds");
    const bool rows_ok = max_k_len % VEC == 0 && nvec <= 64 * 4 && (reinterpret_cast<uintptr_t>(scores) & 15u) == 0 &&
                         scale > 0.0f;
    if (rows_ok) {
        const dim3 grid((unsigned)((max_q_len + 3) / 4), (unsigned)head_num, (unsigned)batch), block(256);
        const float scale_log2e = scale * 1.4426950408889634f;
#define ISP_SOFTMAX_ROWS(N)                                                                              \
    hipLaunchKernelGGL((masked_scaled_softmax_rows<T, N>), grid, block, 0, nullptr, scores, history_length, \
                       input_length, context_length, max_q_len, max_k_len, scale_log2e)
        if (nvec <= 64) ISP_SOFTMAX_ROWS(1);
        else if (nvec <= 128) ISP_SOFTMAX_ROWS(2);
        else ISP_SOFTMAX_ROWS(4);
#undef ISP_SOFTMAX_ROWS
    } else {
        hipLaunchKernelGGL((masked_scaled_softmax<T>), dim3((unsigned)max_q_len, (unsigned)head_num, (unsigned)batch),
                           dim3(256), 0, nullptr, scores, history_length, input_length, context_length, head_num,
                           max_q_len, max_k_len, scale);
    }
    CHECK(hipGetLastError());
}

template void launch_masked_scaled_softmax<float>(float*, const int*, const int*, const int*, int, int, int, int, float);
template void launch_masked_scaled_softmax<half>(half*, const int*, const int*, const int*, int, int, int, int, float);

}  // namespace isp_layers

namespace {

template <typename T>
TensorWrapper<T>* as(Tensor* t, const char* name) {
    LLM_CHECK_WITH_INFO(t->dtype == getTensorType<T>(), std::string(name) + " has the wrong element type");
    return static_cast<TensorWrapper<T>*>(t);
}

// Whether a weight declared [rows, cols] is stored [out_features, in_features] (the reference's
// constructor, layer_weights.cc:23,26,36,38) or [in_features, out_features] (the non-transposed case
// of its GEMM wrapper, linear.cu:36-39).  A square weight is taken to be [out, in].
template <typename T>
bool stored_out_in(const BaseWeight<T>& w, int out_features, int in_features, const char* name) {
    LLM_CHECK_WITH_INFO(w.data != nullptr && w.shape.size() == 2, std::string(name) + " weight is not loaded");
    if (w.shape[0] == out_features && w.shape[1] == in_features) return true;
    LLM_CHECK_WITH_INFO(w.shape[0] == in_features && w.shape[1] == out_features,
                        std::string(name) + " weight has the wrong shape");
    return false;
}

}  // namespace

template <typename T>
LlamaContextDecoderLayer<T>::LlamaContextDecoderLayer(int head_num, int kv_head_num, int head_size, int inter_size,
                                                      const LLaMAAttentionStaticParams& attn_params,
                                                      float rmsnorm_eps, BaseAllocator* allocator)
    : head_num_(head_num),
      kv_head_num_(kv_head_num),
      head_size_(head_size),
      inter_size_(inter_size),
      hidden_(head_num * head_size),
      attn_params_(attn_params),
      eps_(rmsnorm_eps),
      allocator_(allocator) {
    LLM_CHECK_WITH_INFO(allocator != nullptr, "the layer needs an allocator for its buffers");
    LLM_CHECK_WITH_INFO(head_num > 0 && kv_head_num > 0 && head_num % kv_head_num == 0 && head_size > 0 && inter_size > 0,
                        "inconsistent layer dimensions");
    gemm_.reset(new isp_layers::GemmEngine(allocator));
    const char* attention = std::getenv("ISP_LAYERS_ATTENTION");
    fused_attention_ = std::is_same<T, half>::value &&
                       isp_layers::fused_context_attention_supports(head_size, head_num, kv_head_num) &&
                       !(attention != nullptr && std::strcmp(attention, "padded") == 0);
}

template <typename T>
LlamaContextDecoderLayer<T>::~LlamaContextDecoderLayer() {
    freeBuf();
}

template <typename T>
size_t LlamaContextDecoderLayer<T>::workspaceBytes(const LLaMAAttentionDynParams& d) const {
    const size_t tokens = d.num_tokens, b = d.batch_size, q = d.max_q_len, k = d.max_k_len, hs = head_size_;
    size_t elems = tokens * (head_num_ + 2 * kv_head_num_) * hs + b * head_num_ * q * hs + tokens * head_num_ * hs +
                   tokens * 2 * inter_size_ + tokens * inter_size_;
    if (!fused_attention_) elems += 2 * b * head_num_ * k * hs + b * head_num_ * q * k + b * head_num_ * q * hs;
    return elems * sizeof(T);
}

template <typename T>
void LlamaContextDecoderLayer<T>::allocForForward(const LLaMAAttentionDynParams& d) {
    const size_t tokens = d.num_tokens, b = d.batch_size, q = d.max_q_len, k = d.max_k_len, hs = head_size_;
    bool fresh_padding = false;   // a padded buffer is new (or laid out for other extents): zero it
    auto ensure = [this](T*& buf, size_t& capacity, size_t elems) {
        if (elems <= capacity) return false;
        if (buf) allocator_->UnifyFree(buf, false);
        buf = static_cast<T*>(allocator_->UnifyMalloc(nullptr, elems * sizeof(T), false));
        capacity = elems;
        return true;
    };
    ensure(qkv_buf_, capacity_[0], tokens * (head_num_ + 2 * kv_head_num_) * hs);
    fresh_padding |= ensure(q_buf_, capacity_[1], b * head_num_ * q * hs);
    if (!fused_attention_) {
        fresh_padding |= ensure(k_all_, capacity_[2], b * head_num_ * k * hs);
        fresh_padding |= ensure(v_all_, capacity_[3], b * head_num_ * k * hs);
        ensure(scores_, capacity_[4], b * head_num_ * q * k);
        ensure(ctx_, capacity_[5], b * head_num_ * q * hs);
    }
    ensure(ctx_packed_, capacity_[6], tokens * head_num_ * hs);
    ensure(gate_up_, capacity_[7], tokens * 2 * inter_size_);
    ensure(act_, capacity_[8], tokens * inter_size_);
    // padded positions of q (and the k / v rows past a sequence's context) are never written by the
    // kernels; they only meet zero probabilities or discarded rows, but must not hold NaN patterns --
    // nor what an earlier call with other extents left at positions that are padding now
    const bool relaid = d.batch_size != allocated_.batch_size || d.max_q_len != allocated_.max_q_len ||
                        (!fused_attention_ && d.max_k_len != allocated_.max_k_len);
    if (fresh_padding || relaid) {
        CHECK(hipMemsetAsync(q_buf_, 0, b * head_num_ * q * hs * sizeof(T), nullptr));
        if (!fused_attention_) {
            CHECK(hipMemsetAsync(k_all_, 0, b * head_num_ * k * hs * sizeof(T), nullptr));
            CHECK(hipMemsetAsync(v_all_, 0, b * head_num_ * k * hs * sizeof(T), nullptr));
        }
    }
    allocated_ = d;
}

template <typename T>
void LlamaContextDecoderLayer<T>::freeBuf() {
    T** all[] = {&qkv_buf_, &q_buf_, &k_all_, &v_all_, &scores_, &ctx_, &ctx_packed_, &gate_up_, &act_};
    for (int i = 0; i < 9; i++) {
        if (*all[i]) allocator_->UnifyFree(*all[i], false);
        *all[i] = nullptr;
        capacity_[i] = 0;
    }
    allocated_ = LLaMAAttentionDynParams();
}

template <typename T>
void LlamaContextDecoderLayer<T>::forward(TensorMap& inputs, LlamaLayerWeight<T>& weights,
                                          LayerNormWeight<T>& next_attn_norm, TensorMap& outputs,
                                          const LLaMAAttentionDynParams& dyn) {
    TensorWrapper<T>* decoder_input = as<T>(inputs["decoder_input"], "decoder_input");
    TensorWrapper<T>* residual = as<T>(inputs["decoder_residual"], "decoder_residual");
    TensorWrapper<int>* padding_offset = as<int>(inputs["padding_offset"], "padding_offset");
    TensorWrapper<int>* history_length = as<int>(inputs["history_length"], "history_length");
    TensorWrapper<int>* input_length = as<int>(inputs["input_length"], "input_length");
    TensorWrapper<int>* context_length = as<int>(inputs["context_length"], "context_length");
    TensorWrapper<int>* layer_id = as<int>(inputs["layer_id"], "layer_id");
    TensorWrapper<T>* decoder_output = as<T>(outputs["decoder_output"], "decoder_output");
    TensorWrapper<T>* k_cache = as<T>(outputs["all_k_cache"], "all_k_cache");
    TensorWrapper<T>* v_cache = as<T>(outputs["all_v_cache"], "all_v_cache");

    const int tokens = dyn.num_tokens, batch = dyn.batch_size, max_q = dyn.max_q_len, max_k = dyn.max_k_len;
    const int hs = head_size_, heads = head_num_ + 2 * kv_head_num_;
    LLM_CHECK_WITH_INFO(decoder_input->shape.size() == 2 && decoder_input->shape[0] == tokens &&
                            decoder_input->shape[1] == hidden_,
                        "decoder_input should be [num_tokens, hidden]");
    LLM_CHECK_WITH_INFO(residual->shape == decoder_input->shape && decoder_output->shape == decoder_input->shape,
                        "decoder_residual / decoder_output should match decoder_input");
    LLM_CHECK_WITH_INFO(padding_offset->shape.size() == 2 && padding_offset->shape[0] == batch &&
                            padding_offset->shape[1] == max_q,
                        "padding_offset should be [batch, max_q_len]");
    LLM_CHECK_WITH_INFO(history_length->shape[0] == batch && input_length->shape[0] == batch &&
                            context_length->shape[0] == batch,
                        "length tensors should hold one entry per sequence");
    LLM_CHECK_WITH_INFO(k_cache->shape.size() == 5 && k_cache->shape[3] >= max_k, "KV cache shorter than max_k_len");
    LLM_CHECK_WITH_INFO(next_attn_norm.gamma != nullptr && weights.ffn_norm_weight.gamma != nullptr,
                        "norm weights are not loaded");
    if (tokens == 0) return;
    allocForForward(dyn);   // grow-only: allocates only what this call needs beyond what earlier calls left

    const hipDataType lt = isp_layers::LtType<T>::value;
    const DataType dt = getTensorType<T>();
    auto& attn = weights.self_attn_weight;
    auto& ffn = weights.ffn_weight;

    // 1. fused QKV projection: [tokens, hidden] x Wqkv -> [tokens, heads, hs]   (linear.cu:7)
    const bool qkv_oi = stored_out_in(attn.qkv, heads * hs, hidden_, "qkv");
    gemm_->matmul(lt, decoder_input->data, attn.qkv.data, qkv_buf_, tokens, heads * hs, hidden_, qkv_oi, hidden_,
                  qkv_oi ? hidden_ : heads * hs, heads * hs);
    // 2. bias + RoPE + transpose / re-pad of q, and k, v straight into the cache
    TensorWrapper<T> qkv_t(GPU, dt, {tokens, heads, hs}, qkv_buf_);
    TensorWrapper<T> q_t(GPU, dt, {batch, head_num_, max_q, hs}, q_buf_);
    launchAddFusedQKVBiasTransposeRoPEAndConcatKV(&q_t, &qkv_t, attn.qkv, padding_offset, history_length,
                                                  input_length, layer_id, k_cache, v_cache, attn_params_);
    if (fused_attention_) {
        // 3-5. attention over the cache itself, straight to packed [tokens, heads, hs]: one kernel
        LLM_CHECK_WITH_INFO(k_cache->shape[2] == kv_head_num_ && k_cache->shape[4] == hs && v_cache->shape == k_cache->shape,
                            "k / v cache extents should match the layer's");
        const int layer = layer_id->getVal();
        LLM_CHECK_WITH_INFO(layer >= 0 && layer < k_cache->shape[0] && k_cache->shape[1] >= batch, "layer id or batch outside the cache");
        const size_t slice = (size_t)layer * k_cache->shape[1] * k_cache->shape[2] * k_cache->shape[3] * k_cache->shape[4];
        if constexpr (std::is_same<T, half>::value)
            isp_layers::launch_fused_context_attention(q_buf_, k_cache->data + slice, v_cache->data + slice, ctx_packed_,
                                                       history_length->data, input_length->data, context_length->data,
                                                       batch, head_num_, kv_head_num_, hs, max_q, max_k, k_cache->shape[3],
                                                       tokens, 1.0f / std::sqrt((float)hs));
    } else {
        // 3. cache -> k, v of every query head over the whole context (GQA broadcast)
        TensorWrapper<T> k_all_t(GPU, dt, {batch, head_num_, max_k, hs}, k_all_);
        TensorWrapper<T> v_all_t(GPU, dt, {batch, head_num_, max_k, hs}, v_all_);
        launchRepeatKVCache(k_cache, v_cache, context_length, layer_id, &k_all_t, &v_all_t);
        // 4. attention: scores = q k^T, masked softmax, ctx = p v   (batched GEMMs, linear.cu:67-109)
        const int bh = batch * head_num_;
        gemm_->matmul(lt, q_buf_, k_all_, scores_, max_q, max_k, hs, true, hs, hs, max_k, bh, (long long)max_q * hs,
                      (long long)max_k * hs, (long long)max_q * max_k);
        isp_layers::launch_masked_scaled_softmax(scores_, history_length->data, input_length->data, context_length->data,
                                                 batch, head_num_, max_q, max_k, 1.0f / std::sqrt((float)hs));
        gemm_->matmul(lt, scores_, v_all_, ctx_, max_q, hs, max_k, false, max_k, hs, hs, bh, (long long)max_q * max_k,
                      (long long)max_k * hs, (long long)max_q * hs);
        // 5. [batch, heads, max_q, hs] -> packed [tokens, heads, hs]
        TensorWrapper<T> ctx_t(GPU, dt, {batch, head_num_, max_q, hs}, ctx_);
        TensorWrapper<T> packed_t(GPU, dt, {tokens, head_num_, hs}, ctx_packed_);
        launchTransposeOutRemovePadding(&ctx_t, padding_offset, &packed_t);
    }
    // 6. output projection into decoder_input's storage (its contents are no longer needed)   (linear.cu:8)
    const bool o_oi = stored_out_in(attn.output, hidden_, hidden_, "attention output");
    gemm_->matmul(lt, ctx_packed_, attn.output.data, decoder_input->data, tokens, hidden_, hidden_, o_oi, hidden_,
                  hidden_, hidden_);
    // 7. residual += attn (+ bias); decoder_input := RMSNorm by ffn_norm
    launchFusedAddBiasResidualRMSNorm(residual, decoder_input, attn.output, weights.ffn_norm_weight.gamma, eps_);
    // 8. gate / up projection -> [tokens, 2, inter]   (linear.cu:14)
    const bool gu_oi = stored_out_in(ffn.gateAndup, 2 * inter_size_, hidden_, "gate/up");
    gemm_->matmul(lt, decoder_input->data, ffn.gateAndup.data, gate_up_, tokens, 2 * inter_size_, hidden_, gu_oi,
                  hidden_, gu_oi ? hidden_ : 2 * inter_size_, 2 * inter_size_);
    // 9. SwiGLU
    TensorWrapper<T> gate_up_t(GPU, dt, {tokens, 2, inter_size_}, gate_up_);
    TensorWrapper<T> act_t(GPU, dt, {tokens, inter_size_}, act_);
    launchAct(&gate_up_t, &act_t);
    // 10. down projection   (linear.cu:15)
    const bool down_oi = stored_out_in(ffn.down, hidden_, inter_size_, "down");
    gemm_->matmul(lt, act_, ffn.down.data, decoder_output->data, tokens, hidden_, inter_size_, down_oi, inter_size_,
                  down_oi ? inter_size_ : hidden_, hidden_);
    // 11. residual += ffn (+ bias); decoder_output := RMSNorm by the next layer's attention norm
    launchFusedAddBiasResidualRMSNorm(residual, decoder_output, ffn.down, next_attn_norm.gamma, eps_);
}

template class LlamaContextDecoderLayer<float>;
template class LlamaContextDecoderLayer<half>;
