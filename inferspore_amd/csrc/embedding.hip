// Input-embedding gather for gfx950: out[t, :] = table[ids[t], :].
//
// Semantics: src/kernels/input_embedding.cu:14-21.  It is a raw row copy, so one kernel serves every
// element type (the row is handled as bytes) and the result is bit-exact by construction.
// Design: one wave per token row; the token id is read once per row into a scalar register (the
// reference re-reads ids[] and does a div/mod for every 2-byte element); the row moves as 16-byte
// vectors with eight loads in flight per lane; four rows per workgroup.
#include "isp_common.h"

namespace isp {

template <int UNROLL>
__global__ __launch_bounds__(kBlock) void gather_rows_vec(const int32_t* __restrict__ ids,
                                                          char* __restrict__ out,
                                                          const char* __restrict__ table, int tokens,
                                                          unsigned row_vec, int vocab) {
    const int wave = threadIdx.x / kWave;
    const int lane = threadIdx.x % kWave;
    const int row = blockIdx.x * (kBlock / kWave) + wave;
    if (row >= tokens) return;  // whole wave leaves together; no barrier follows
    const int id = __builtin_amdgcn_readfirstlane(ids[row]);
    const bool in_range = vocab <= 0 || (id >= 0 && id < vocab);
    const size_t row_bytes = (size_t)row_vec * 16u;
    const char* src = table + (size_t)(in_range ? id : 0) * row_bytes;
    char* dst = out + (size_t)row * row_bytes;
    for (unsigned v0 = lane; v0 < row_vec; v0 += kWave * UNROLL) {
        vec16 buf[UNROLL];
#pragma unroll
        for (int k = 0; k < UNROLL; k++) {
            const unsigned v = v0 + k * kWave;
            if (v < row_vec) {
                if (in_range) {
                    buf[k] = load16_stream(src + (size_t)v * 16u);
                } else {
                    buf[k].w[0] = buf[k].w[1] = buf[k].w[2] = buf[k].w[3] = 0u;
                }
            }
        }
#pragma unroll
        for (int k = 0; k < UNROLL; k++) {
            const unsigned v = v0 + k * kWave;
            if (v < row_vec) store16(dst + (size_t)v * 16u, buf[k]);
        }
    }
}

// Rows that are not a whole number of aligned 16-byte vectors: one workgroup per row, byte copies.
__global__ __launch_bounds__(kBlock) void gather_rows_bytes(const int32_t* ids, char* out,
                                                            const char* table, int tokens,
                                                            size_t row_bytes, int vocab) {
    const int row = blockIdx.x;
    const int id = ids[row];
    const bool in_range = vocab <= 0 || (id >= 0 && id < vocab);
    const char* src = table + (size_t)(in_range ? id : 0) * row_bytes;
    char* dst = out + (size_t)row * row_bytes;
    for (size_t i = threadIdx.x; i < row_bytes; i += kBlock) dst[i] = in_range ? src[i] : (char)0;
}

static int embedding(const int32_t* ids, void* out, const void* table, int tokens, int hidden,
                     int vocab, int elem_size, hipStream_t s) {
    if (tokens < 0 || hidden < 0 || vocab < 0) return ISP_ERR_BAD_SHAPE;
    if (tokens == 0 || hidden == 0) return ISP_OK;
    ISP_REQUIRE_PTR(ids);
    ISP_REQUIRE_PTR(out);
    ISP_REQUIRE_PTR(table);
    const size_t row_bytes = (size_t)hidden * (size_t)elem_size;
    hipError_t e;
    if (row_bytes % 16 == 0 && aligned16(out) && aligned16(table)) {
        constexpr int ROWS = kBlock / kWave;
        dim3 grid((unsigned)((tokens + ROWS - 1) / ROWS));
        hipLaunchKernelGGL((gather_rows_vec<8>), grid, dim3(kBlock), 0, s, ids,
                           static_cast<char*>(out), static_cast<const char*>(table), tokens,
                           (unsigned)(row_bytes / 16), vocab);
        e = hipGetLastError();
    } else {
        hipLaunchKernelGGL(gather_rows_bytes, dim3((unsigned)tokens), dim3(kBlock), 0, s, ids,
                           static_cast<char*>(out), static_cast<const char*>(table), tokens,
                           row_bytes, vocab);
        e = hipGetLastError();
    }
    return note_launch(e);
}

}  // namespace isp

extern "C" {

int isp_embedding_f16(const int32_t* ids, void* out, const void* table, int tokens, int hidden,
                      int vocab, isp_stream_t stream) {
    return isp::embedding(ids, out, table, tokens, hidden, vocab, 2, static_cast<hipStream_t>(stream));
}

int isp_embedding_f32(const int32_t* ids, void* out, const void* table, int tokens, int hidden,
                      int vocab, isp_stream_t stream) {
    return isp::embedding(ids, out, table, tokens, hidden, vocab, 4, static_cast<hipStream_t>(stream));
}

}  // extern "C"
