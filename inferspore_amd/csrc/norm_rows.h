// Device code shared by the RMSNorm kernels (norm.hip: the general kernel and the launchers; norm_few_rows.hip:
// the kernels that launches of a few rows -- all of whose waves are resident at once -- take).  The two live in separate translation units because they are
// compiled differently: the few-rows kernels with their arguments preloaded into scalar registers at wave
// start, the general kernel without.
#pragma once

#include "isp_common.h"

namespace isp {

// One row is handled by WPR waves (ROW_THREADS = 64 * WPR lanes); a workgroup of BLOCK threads
// (256, 512 or 1024, at least one row) carries BLOCK / ROW_THREADS rows.  Each lane owns NV 16-byte
// vectors of the row, strided by ROW_THREADS so that every load instruction of a wave covers 1 KiB
// of contiguous memory.  ST is the store kind of the two outputs (non-temporal by default).
constexpr int norm_block(int wpr) { return kWave * wpr > kBlock ? kWave * wpr : kBlock; }

// p[0] + ... + p[N-1] as a balanced binary tree, neighbours first; N a power of two.
template <int N>
__device__ __forceinline__ float tree_sum(const float* p) {
    if constexpr (N == 1) {
        return p[0];
    } else {
        return tree_sum<N / 2>(p) + tree_sum<N / 2>(p + N / 2);
    }
}

// The order of the memory operations is the design, and each step of it is measured (2048 x 4096 fp16
// with residual and bias, 67 MB per launch, one round of waves; alternating builds on one device):
//   1. all streamed vectors of the lane are requested at kernel entry;
//   2. nothing is computed or requested until ALL of them have arrived (starting on the first vector
//      while the others are in flight: 12.9 us instead of 11.0 us);
//   3. bias is requested only then, one vector at a time, where it is consumed, and gamma after the
//      row has been summed (either of them requested together with the rows, or both bias vectors
//      at once: 12.6-12.8 us -- every workgroup then hits the same few L2 lines at the same time);
//   4. every store is issued at the very end, behind the barrier, after gamma has arrived (the
//      residual stored inside the loop, as soon as it is known: 11.7 us; a store followed by a
//      wait for a later load also makes the wave wait for the store's acknowledgement, because
//      loads and stores share one in-order counter).
// The common factor of 2-4: the device reaches its best rate when the launch first reads and then
// writes; writes that start while most reads are still queued cost more than the idle registers.
// The opposite order -- start on each vector as it arrives, store the residual as soon as it is known
// -- stays selectable (kNormStreamingOrder, an internal flag bit the launcher sets from a tuning
// knob): with several rounds of waves it measured within 1 % of the order above for 16-bit rows and
// plain RMSNorm, and 8-12 % slower for 32-bit rows with a residual.  Same bits under both.
constexpr unsigned kNormStreamingOrder = 0x80000000u;
// Step 3 is more than a way to fetch the bias: the cache round trip it puts between the arrival of a wave's rows
// and its first store is what keeps the early waves' stores out of the late waves' reads.  A call WITHOUT a bias
// (every LLaMA layer: its projections have none) loses that wait, and where the launch is about one round of waves
// it measured 10-27 % slower than the same call with a bias (2977 x 4096 fp16 with a residual: 18.6 against
// 16.2 us; 2048 rows 12.7 against 11.2; fp32 1024-2304 rows alike).  kNormPacingLoad restores it: in place of the
// absent bias vector the wave requests its gamma vector there and waits for it (the value is requested again
// where it is used; both are cache hits).  With it the call without a bias takes what the call with one takes.
// The launcher sets it for residual-without-bias launches that fit one round of waves and read more than 24 MiB;
// below that size, over several rounds of waves, and for plain RMSNorm it measured 1-12 % slower and stays off.
constexpr unsigned kNormPacingLoad = 0x40000000u;
constexpr unsigned kNormInternalFlags = kNormStreamingOrder | kNormPacingLoad;

// Which operands exist: known only at run time (the general kernel: uniform scalar branches), or fixed at
// compile time for the kernels that launches of a few rows take (fused_norm_few_rows).
constexpr int kOpsRuntime = -1, kOpsNone = 0, kOpsResidual = 1, kOpsResidualBias = 2;

template <typename T, int NV, int WPR, int ST, int BLOCK, int OPS>
__device__ __forceinline__ void norm_rows_body(T* residual, T* out, const T* bias, const T* gamma, float eps,
                                               int tokens, int hidden, unsigned flags) {
    constexpr int VEC = Elem<T>::kVec;
    constexpr int ROW_THREADS = kWave * WPR;
    static_assert(BLOCK >= norm_block(WPR) && BLOCK % ROW_THREADS == 0, "workgroup must hold whole rows");
    constexpr int ROWS = BLOCK / ROW_THREADS;

    const int slot = threadIdx.x / ROW_THREADS;
    const int lane = threadIdx.x % ROW_THREADS;
    const int row = blockIdx.x * ROWS + slot;
    const bool live = row < tokens;  // uniform within a wave
    const int nvec = hidden / VEC;
    const bool has_res = OPS == kOpsRuntime ? residual != nullptr : OPS >= kOpsResidual;  // uniform: scalar branches
    const bool has_bias = OPS == kOpsRuntime ? bias != nullptr : OPS == kOpsResidualBias;
    const bool literal_order = OPS == kOpsRuntime && (flags & ISP_NORM_RESIDUAL_EXCLUDES_BIAS) != 0;
    const bool streaming = OPS == kOpsRuntime && (flags & kNormStreamingOrder) != 0;
    const bool pacing = OPS == kOpsRuntime && (flags & kNormPacingLoad) != 0;
    const size_t base = (size_t)(live ? row : 0) * (size_t)hidden;
    T* out_row = out + base;
    T* rsd_row = residual + base;  // dereferenced only when has_res

    // the small operands' addresses are fetched with the other arguments at kernel entry (left alone, the
    // compiler fetches the gamma pointer only where it is first used: a scalar round trip behind the row's arrival)
    asm volatile("" : : "s"(gamma), "s"(bias));
    vec16 vo[NV], vr[NV];
    bool ok[NV];
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int vi = lane + j * ROW_THREADS;
        ok[j] = live && vi < nvec;
        if (ok[j]) {
            vo[j] = load16_stream(out_row + (size_t)vi * VEC);
            if (has_res) vr[j] = load16_stream(rsd_row + (size_t)vi * VEC);
        }
    }
    // step 2: the empty asm uses the loaded registers (so the wait for them is placed here) and
    // nothing that touches memory may be moved across it
    if (!streaming) {
#pragma unroll
        for (int j = 0; j < NV; j++) asm volatile("" : "+v"(vo[j].w[0]), "+v"(vr[j].w[0]) : : "memory");
    }

    float x[NV][VEC];
    float part[NV];  // sum of squares of each of this lane's vectors
#pragma unroll
    for (int j = 0; j < NV; j++) {
        part[j] = 0.0f;
        if (ok[j]) {
            const int vi = lane + j * ROW_THREADS;
            vec16 vb;
            if (has_bias) vb = load16(bias + (size_t)vi * VEC);
            else if (pacing) {
                // no bias to wait for: wait for this vector's gamma instead (see kNormPacingLoad)
                vb = load16(gamma + (size_t)vi * VEC);
                asm volatile("" : "+v"(vb.w[0]) : : "memory");
            }
            asm volatile("" ::: "memory");  // step 3: the next vector's bias is not requested early
            if (has_res) Elem<T>::sum(vo[j], vr[j], x[j]);
            else Elem<T>::unpack(vo[j], x[j]);
            if (has_res && literal_order) {
                // the reference's literal order stores the residual before the bias is added; that
                // mode keeps its store here (x does not survive the addition of the bias)
                store16_sel<ST>(rsd_row + (size_t)vi * VEC, Elem<T>::pack(x[j]));
            }
            if (has_bias) Elem<T>::accumulate(vb, x[j]);
            // x is stored (rounded to T) and also used further in fp32: the value is fixed in its
            // register here so that the rounding of the store cannot be merged with this sum
#pragma unroll
            for (int e = 0; e < VEC; e++) x[j][e] = Elem<T>::pinned(x[j][e]);
            if (has_res && streaming && !literal_order)
                store16_sel<ST>(rsd_row + (size_t)vi * VEC, Elem<T>::pack_pinned(x[j]));
            // one product and then fused multiply-adds in element order: no freedom for the compiler
            // in how it contracts the sum, so every instantiation associates it the same way
            float p = x[j][0] * x[j][0];
#pragma unroll
            for (int e = 1; e < VEC; e++) p = __fmaf_rn(x[j][e], x[j][e], p);
            part[j] = p;
        }
        // with one or two vectors per lane each is reduced over the wave as soon as it is summed,
        // underneath the round trip of the next bias vector
        if (NV <= 2) part[j] = wave_sum(part[j]);
    }

    // gamma is requested once this lane's part of the row has been summed: the L2 round trip then
    // overlaps the reduction and the barrier instead of following them
    vec16 vg[NV];
#pragma unroll
    for (int j = 0; j < NV; j++) {
        if (ok[j]) vg[j] = load16(gamma + (size_t)(lane + j * ROW_THREADS) * VEC);
    }

    // The row sum is the balanced binary tree over the vector index, lowest bit first: lanes of a wave
    // (index bits 0-5, wave_sum), then the waves of the row (next bits), then this lane's own vectors
    // (top bits); absent vectors add exact zeros.  That tree is the same however the row is split
    // over waves and vectors per lane, so the result does not depend on the launch configuration --
    // a row gives the same bits in a batch of 1 and in a batch of 16384.
    if (NV > 2) {
#pragma unroll
        for (int j = 0; j < NV; j++) part[j] = wave_sum(part[j]);
    }
    if (WPR > 1) {
        __shared__ float partial[NV][BLOCK / kWave];
        const int wave = threadIdx.x / kWave;
        if ((threadIdx.x % kWave) == 0) {
#pragma unroll
            for (int j = 0; j < NV; j++) partial[j][wave] = part[j];
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < NV; j++) part[j] = tree_sum<WPR>(&partial[j][slot * WPR]);
    }
    const float total = tree_sum<NV>(part);
    const float inv = rsqrtf(total / (float)hidden + eps);

    // step 4: gamma has arrived before the first store is issued, so no wait below falls behind a store
#pragma unroll
    for (int j = 0; j < NV; j++) asm volatile("" : "+v"(vg[j].w[0]) : : "memory");
    if (has_res && !literal_order && !streaming) {
#pragma unroll
        for (int j = 0; j < NV; j++) {
            if (ok[j])
                store16_sel<ST>(rsd_row + (size_t)(lane + j * ROW_THREADS) * VEC, Elem<T>::pack_pinned(x[j]));
        }
    }
#pragma unroll
    for (int j = 0; j < NV; j++) {
        if (ok[j]) {
            float y[VEC];
            Elem<T>::scale(vg[j], x[j], y);
#pragma unroll
            for (int e = 0; e < VEC; e++) y[e] *= inv;
            store16_sel<ST>(out_row + (size_t)(lane + j * ROW_THREADS) * VEC, Elem<T>::pack(y));
        }
    }
}

// A few-rows kernel (norm_few_rows.hip): the same row body with the operand set fixed at compile time.
template <typename T>
using NormFewKernel = void (*)(T*, T*, const T*, const T*, float, int, int);

// The few-rows instantiation for (waves per row, vectors per lane, store kind, operands), or nullptr: one
// vector per lane with any number of waves per row, two only with 16 waves (rows are split as far as they
// go before a lane takes a second vector); plain or non-temporal stores.  Defined for float and __half.
template <typename T>
NormFewKernel<T> norm_few_variant(int wpr, int nv, int st, int ops);

}  // namespace isp
