// SwiGLU activation for gfx950: out[t, i] = silu(in[t, 0, i]) * in[t, 1, i].
//
// Semantics: src/kernels/act_kernel.cu:6-10,25-33 (silu(x) = x / (1 + expf(-x)) in fp32, product in
// fp32) with a single rounding to the storage type, as in tests/unittests/test_act.cu:13-25.
// Design: the output is treated as one flat array of 16-byte vectors, so every lane of every wave
// is busy whatever the row length (the reference's one-block-per-token loop leaves decode batches
// with 256 half2-wide blocks); each lane keeps UNROLL gate/up vector pairs in flight.
#include "isp_common.h"

namespace isp {

__device__ __forceinline__ float silu_exact(float x) { return x / (1.0f + expf(-x)); }

// exp through the hardware exp2 and a hardware reciprocal: relative error of a few 1e-7, three
// orders of magnitude below half an fp16 ulp, so the rounded fp16 result matches the exact form
// except on rounding ties.
__device__ __forceinline__ float silu_fast(float x) {
    const float e = __builtin_amdgcn_exp2f(-1.4426950408889634f * x);
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

template <typename T>
__device__ __forceinline__ float silu_for(float x);
template <>
__device__ __forceinline__ float silu_for<float>(float x) { return silu_exact(x); }
template <>
__device__ __forceinline__ float silu_for<__half>(float x) { return silu_fast(x); }

// Single-wave workgroups: 80.8 against 83.2 us with 256 threads at 8192 x 11008 fp16, equal from 2977 rows down.
template <typename T, int UNROLL, int ST>
__global__ __launch_bounds__(kWave) void swiglu_vec(const T* __restrict__ in, T* __restrict__ out,
                                                    unsigned total_vec, unsigned vec_per_row) {
    constexpr int VEC = Elem<T>::kVec;
    const unsigned first = blockIdx.x * (unsigned)(kWave * UNROLL) + threadIdx.x;
    vec16 g[UNROLL], u[UNROLL];
    bool ok[UNROLL];
#pragma unroll
    for (int k = 0; k < UNROLL; k++) {
        const unsigned v = first + k * kWave;
        ok[k] = v < total_vec;
        if (ok[k]) {
            const unsigned t = v / vec_per_row;
            const size_t gate = ((size_t)v + (size_t)t * vec_per_row) * VEC;  // row t starts at 2 t I
            g[k] = load16_stream(in + gate);
            u[k] = load16_stream(in + gate + (size_t)vec_per_row * VEC);
        }
    }
#pragma unroll
    for (int k = 0; k < UNROLL; k++) {
        if (ok[k]) {
            const unsigned v = first + k * kWave;
            float a[VEC], b[VEC], y[VEC];
            Elem<T>::unpack(g[k], a);
            Elem<T>::unpack(u[k], b);
#pragma unroll
            for (int e = 0; e < VEC; e++) y[e] = silu_for<T>(a[e]) * b[e];
            store16_sel<ST>(out + (size_t)v * VEC, Elem<T>::pack(y));
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void swiglu_generic(const T* in, T* out, size_t total,
                                                         unsigned inter) {
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < total;
         i += (size_t)gridDim.x * kBlock) {
        const size_t t = i / inter;
        const size_t gate = i + t * inter;
        const float a = Elem<T>::to_f32(in[gate]);
        const float b = Elem<T>::to_f32(in[gate + inter]);
        out[i] = Elem<T>::from_f32(silu_for<T>(a) * b);  // same formulation as swiglu_vec: bit-identical
    }
}

template <typename T>
static int swiglu(const void* in_, void* out_, int tokens, int inter, hipStream_t s) {
    if (tokens < 0 || inter < 0) return ISP_ERR_BAD_SHAPE;
    if (tokens == 0 || inter == 0) return ISP_OK;
    ISP_REQUIRE_PTR(in_);
    ISP_REQUIRE_PTR(out_);
    const T* in = static_cast<const T*>(in_);
    T* out = static_cast<T*>(out_);
    constexpr int VEC = Elem<T>::kVec;
    const size_t total = (size_t)tokens * (size_t)inter;
    const size_t total_vec = total / VEC;
    hipError_t e;
    // 32-bit vector indices in the kernel: leave room for the last workgroup's overshoot
    if (inter % VEC == 0 && aligned16(in) && aligned16(out) && total_vec < 0xffff0000ull) {
        int unroll = tuning(ISP_TUNE_SWIGLU_UNROLL);
        if (unroll != 1 && unroll != 2 && unroll != 4) unroll = 1;
        // non-temporal stores: equal to or 1-2 % ahead of the write-through form at every size from 256 to 8192
        // rows of 11008 in both precisions, 5-10 % ahead of ordinary stores from 1024 rows up
        const int kind = store_kind(tuning(ISP_TUNE_SWIGLU_STORE), kStoreStream);
        const size_t per_block = (size_t)kWave * unroll;
        const dim3 grid((unsigned)((total_vec + per_block - 1) / per_block)), block(kWave);
        const unsigned nv = (unsigned)total_vec, vpr = (unsigned)(inter / VEC);
#define ISP_SWIGLU_LAUNCH(U, K) \
    hipLaunchKernelGGL((swiglu_vec<T, U, K>), grid, block, 0, s, in, out, nv, vpr)
#define ISP_SWIGLU_KIND(U)                                               \
    do {                                                                 \
        if (kind == kStoreThrough) ISP_SWIGLU_LAUNCH(U, kStoreThrough);  \
        else if (kind == kStoreStream) ISP_SWIGLU_LAUNCH(U, kStoreStream); \
        else ISP_SWIGLU_LAUNCH(U, kStorePlain);                          \
    } while (0)
        if (unroll == 1) ISP_SWIGLU_KIND(1);
        else if (unroll == 2) ISP_SWIGLU_KIND(2);
        else ISP_SWIGLU_KIND(4);
#undef ISP_SWIGLU_KIND
#undef ISP_SWIGLU_LAUNCH
        e = hipGetLastError();
    } else {
        size_t blocks = (total + kBlock - 1) / kBlock;
        if (blocks > 65536) blocks = 65536;
        hipLaunchKernelGGL((swiglu_generic<T>), dim3((unsigned)blocks), dim3(kBlock), 0, s, in, out,
                           total, (unsigned)inter);
        e = hipGetLastError();
    }
    return note_launch(e);
}

}  // namespace isp

extern "C" {

int isp_swiglu_f32(const void* in, void* out, int tokens, int inter, isp_stream_t stream) {
    return isp::swiglu<float>(in, out, tokens, inter, static_cast<hipStream_t>(stream));
}

int isp_swiglu_f16(const void* in, void* out, int tokens, int inter, isp_stream_t stream) {
    return isp::swiglu<__half>(in, out, tokens, inter, static_cast<hipStream_t>(stream));
}

}  // extern "C"
