// A plain device-to-device copy of known size.  It has no counterpart in the reference: it exists so
// that profiler byte counters (and the achievable copy bandwidth of the machine) can be calibrated
// against a kernel whose traffic is known exactly -- `bytes` read and `bytes` written.  It uses the
// same access recipe as the production kernels (16-byte vectors, one per lane, non-temporal), in
// single-wave workgroups: 2-4 % faster than 256-thread ones from 64 MiB of traffic up (11.3 against 11.8 us
// at 64 MiB, 78.5 against 80.4 at 512 MiB), equal below.
#include "isp_common.h"

namespace isp {

template <int UNROLL>
__global__ __launch_bounds__(kWave) void copy_vec(char* __restrict__ dst,
                                                   const char* __restrict__ src, size_t nvec) {
    const size_t first = (size_t)blockIdx.x * (kWave * UNROLL) + threadIdx.x;
    vec16 buf[UNROLL];
#pragma unroll
    for (int k = 0; k < UNROLL; k++) {
        const size_t v = first + (size_t)k * kWave;
        if (v < nvec) buf[k] = load16_stream(src + v * 16);
    }
#pragma unroll
    for (int k = 0; k < UNROLL; k++) {
        const size_t v = first + (size_t)k * kWave;
        if (v < nvec) store16_through(dst + v * 16, buf[k]);
    }
}

}  // namespace isp

extern "C" int isp_calibration_copy(void* dst, const void* src, size_t bytes, isp_stream_t stream) {
    if (bytes == 0) return ISP_OK;
    ISP_REQUIRE_PTR(dst);
    ISP_REQUIRE_PTR(src);
    if (bytes % 16 != 0 || !isp::aligned16(dst) || !isp::aligned16(src)) return ISP_ERR_BAD_SHAPE;
    constexpr int UNROLL = 1;  // one vector per lane streams best on this memory system
    const size_t nvec = bytes / 16;
    const size_t per_block = (size_t)isp::kWave * UNROLL;
    const size_t blocks = (nvec + per_block - 1) / per_block;
    if (blocks > 0x7fffffffull) return ISP_ERR_UNSUPPORTED;
    hipLaunchKernelGGL((isp::copy_vec<UNROLL>), dim3((unsigned)blocks), dim3(isp::kWave), 0,
                       static_cast<hipStream_t>(stream), static_cast<char*>(dst),
                       static_cast<const char*>(src), nvec);
    return isp::note_launch(hipGetLastError());
}
