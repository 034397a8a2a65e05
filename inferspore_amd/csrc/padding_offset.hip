// Padding-offset builder for gfx950.
//
// Semantics: the serial loop of src/kernels/cal_paddingoffset.cu:23-44 -- for the tokens of
// sequence b (packed index running over all sequences) padding_offset = sum_{b' < b}(max_q_len -
// len[b']), cum_seqlens[b] = sum_{b' < b} len[b'], cum_seqlens[batch] = total.
// Design: the reference runs this on a single thread; here one workgroup per sequence sums the
// (few) preceding lengths itself and then fills its own token range in parallel, so there is no
// cross-workgroup dependency and the launch is a single wave of latency.
#include "isp_common.h"

namespace isp {

__device__ __forceinline__ int block_sum_int(int v, int* scratch) {
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, kWave);
    if ((threadIdx.x % kWave) == 0) scratch[threadIdx.x / kWave] = v;
    __syncthreads();
    const int total = (scratch[0] + scratch[1]) + (scratch[2] + scratch[3]);
    __syncthreads();
    return total;
}

__global__ __launch_bounds__(kBlock) void padding_offset_kernel(int32_t* padding_offset,
                                                                int32_t* cum_seqlens,
                                                                const int32_t* input_lengths,
                                                                int batch, int max_q_len) {
    __shared__ int scratch[kBlock / kWave];
    const int b = blockIdx.x;
    if (batch == 0) {
        if (threadIdx.x == 0) cum_seqlens[0] = 0;
        return;
    }
    int raw = 0;    // sum of preceding lengths as given
    int count = 0;  // number of offsets written by preceding sequences (negative lengths write none)
    for (int i = threadIdx.x; i < b; i += kBlock) {
        const int len = input_lengths[i];
        raw += len;
        count += len > 0 ? len : 0;
    }
    raw = block_sum_int(raw, scratch);
    count = block_sum_int(count, scratch);
    const int len = input_lengths[b];
    const int offset = b * max_q_len - raw;
    const long long capacity = (long long)batch * (long long)max_q_len;
    for (int i = threadIdx.x; i < len; i += kBlock) {
        const long long ind = (long long)count + i;
        if (ind < capacity) padding_offset[ind] = offset;
    }
    if (threadIdx.x == 0) {
        cum_seqlens[b] = raw;
        if (b == batch - 1) cum_seqlens[batch] = raw + len;
    }
}

}  // namespace isp

extern "C" int isp_cal_padding_offset(int32_t* padding_offset, int32_t* cum_seqlens,
                                      const int32_t* input_lengths, int batch, int max_q_len,
                                      isp_stream_t stream) {
    if (batch < 0 || max_q_len < 0) return ISP_ERR_BAD_SHAPE;
    ISP_REQUIRE_PTR(cum_seqlens);
    if (batch > 0) {
        ISP_REQUIRE_PTR(input_lengths);
        if (max_q_len > 0) ISP_REQUIRE_PTR(padding_offset);
    }
    hipLaunchKernelGGL(isp::padding_offset_kernel, dim3((unsigned)(batch > 0 ? batch : 1)),
                       dim3(isp::kBlock), 0, static_cast<hipStream_t>(stream), padding_offset,
                       cum_seqlens, input_lengths, batch, max_q_len);
    return isp::note_launch(hipGetLastError());
}
