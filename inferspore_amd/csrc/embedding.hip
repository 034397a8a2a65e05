// Input-embedding gather for gfx950: out[t, :] = table[ids[t], :].
//
// Semantics: src/kernels/input_embedding.cu:14-21.  It is a raw row copy, so one kernel serves every
// element type (the row is handled as bytes) and the result is bit-exact by construction.
// Design: the token id is read once per workgroup into a scalar register (the reference re-reads
// ids[] and does a div/mod for every 2-byte element) and the row moves as 16-byte vectors, one
// vector per lane, one 1 KiB chunk of a row per single-wave workgroup -- the access order that streams
// best on this memory system; wave-per-row and workgroup-per-row variants remain selectable for sweeps.
#include "isp_common.h"

namespace isp {

// ROW_THREADS lanes (a wave, or the whole workgroup) share one row; each lane moves UNROLL vectors
// per trip, strided by ROW_THREADS.
template <int ROW_THREADS, int UNROLL, int ST>
__global__ __launch_bounds__(kBlock) void gather_rows_vec(const int32_t* __restrict__ ids,
                                                          char* __restrict__ out,
                                                          const char* __restrict__ table, int tokens,
                                                          unsigned row_vec, int vocab) {
    constexpr int ROWS = kBlock / ROW_THREADS;
    const int slot = threadIdx.x / ROW_THREADS;
    const int lane = threadIdx.x % ROW_THREADS;
    const int row = blockIdx.x * ROWS + slot;
    if (row >= tokens) return;  // whole waves leave together; no barrier follows
    const int id = __builtin_amdgcn_readfirstlane(ids[row]);
    const bool in_range = vocab <= 0 || (id >= 0 && id < vocab);
    const size_t row_bytes = (size_t)row_vec * 16u;
    const char* src = table + (size_t)(in_range ? id : 0) * row_bytes;
    char* dst = out + (size_t)row * row_bytes;
    for (unsigned v0 = lane; v0 < row_vec; v0 += ROW_THREADS * UNROLL) {
        vec16 buf[UNROLL];
#pragma unroll
        for (int k = 0; k < UNROLL; k++) {
            const unsigned v = v0 + k * ROW_THREADS;
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
            const unsigned v = v0 + k * ROW_THREADS;
            if (v < row_vec) store16_sel<ST>(dst + (size_t)v * 16u, buf[k]);
        }
    }
}

// One 16-byte vector per lane: a workgroup is a single wave and moves one 1 KiB chunk of one row.  A wave
// that is its own workgroup starts as soon as any wave slot is free; measured against 256-thread
// workgroups (4 KiB chunks) on 8192 rows of fp16: 4096 wide 22.4 against 23.2 us, 5120 wide (whose third
// 4 KiB chunk is half empty) 28.4 against 29.0, 3072 wide 18.0 against 20.2; 128, 192, 320 ... 512 threads
// all lie between or behind.
template <int ST>
__global__ __launch_bounds__(kWave) void gather_chunks_vec(const int32_t* __restrict__ ids,
                                                           char* __restrict__ out,
                                                           const char* __restrict__ table,
                                                           unsigned chunks_per_row,
                                                           unsigned row_vec, int vocab) {
    const unsigned row = blockIdx.x / chunks_per_row;
    const unsigned v = (blockIdx.x % chunks_per_row) * kWave + threadIdx.x;
    if (v >= row_vec) return;
    const int id = __builtin_amdgcn_readfirstlane(ids[row]);
    const bool in_range = vocab <= 0 || (id >= 0 && id < vocab);
    const size_t row_bytes = (size_t)row_vec * 16u;
    vec16 buf;
    if (in_range) buf = load16_stream(table + (size_t)id * row_bytes + (size_t)v * 16u);
    else buf.w[0] = buf.w[1] = buf.w[2] = buf.w[3] = 0u;
    store16_sel<ST>(out + (size_t)row * row_bytes + (size_t)v * 16u, buf);
}

// Rows that are not a whole number of aligned 16-byte vectors: one workgroup per row, copied in units
// of U (the element size when the pointers allow it, bytes otherwise).
template <typename U>
__global__ __launch_bounds__(kBlock) void gather_rows_units(const int32_t* ids, U* out, const U* table,
                                                            int tokens, size_t row_units, int vocab) {
    const int row = blockIdx.x;
    const int id = ids[row];
    const bool in_range = vocab <= 0 || (id >= 0 && id < vocab);
    const U* src = table + (size_t)(in_range ? id : 0) * row_units;
    U* dst = out + (size_t)row * row_units;
    for (size_t i = threadIdx.x; i < row_units; i += kBlock) dst[i] = in_range ? src[i] : (U)0;
}

template <int ST>
static void launch_gather(int variant, const int32_t* ids, char* o, const char* t, int tokens,
                          unsigned row_vec, int vocab, hipStream_t s) {
    const dim3 block(kBlock);
    const size_t chunks = (row_vec + kWave - 1) / kWave;
    if (variant == 1) {  // one wave per row
        hipLaunchKernelGGL((gather_rows_vec<kWave, 4, ST>), dim3((unsigned)((tokens + 3) / 4)), block, 0, s,
                           ids, o, t, tokens, row_vec, vocab);
    } else if (variant == 2 || (size_t)tokens * chunks > 0x7fffffffull) {  // one workgroup per row
        hipLaunchKernelGGL((gather_rows_vec<kBlock, 2, ST>), dim3((unsigned)tokens), block, 0, s, ids, o, t,
                           tokens, row_vec, vocab);
    } else {  // one 1 KiB chunk of a row per single-wave workgroup, one vector per lane
        hipLaunchKernelGGL((gather_chunks_vec<ST>), dim3((unsigned)((size_t)tokens * chunks)), dim3(kWave), 0,
                           s, ids, o, t, (unsigned)chunks, row_vec, vocab);
    }
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
        // write-through stores from 16 MiB of output up (1-2 % over non-temporal ones); below 8 MiB the plain
        // non-temporal store measured 3-7 % faster (256-1024 rows of 8 KiB); up to 1 MiB (a decode step's rows)
        // ordinary stores, which the L2 acknowledges: 1.93 against 2.14 us for 16 rows
        const size_t written = (size_t)tokens * row_bytes;
        const int kind = store_kind(tuning(ISP_TUNE_EMBED_STORE), written <= ((size_t)1 << 20)   ? kStorePlain
                                                                  : written <= ((size_t)8 << 20) ? kStoreStream
                                                                                                 : kStoreThrough);
        const unsigned row_vec = (unsigned)(row_bytes / 16);
        char* o = static_cast<char*>(out);
        const char* t = static_cast<const char*>(table);
        const int variant = tuning(ISP_TUNE_EMBED_VARIANT);
        if (kind == kStoreThrough) launch_gather<kStoreThrough>(variant, ids, o, t, tokens, row_vec, vocab, s);
        else if (kind == kStoreStream) launch_gather<kStoreStream>(variant, ids, o, t, tokens, row_vec, vocab, s);
        else launch_gather<kStorePlain>(variant, ids, o, t, tokens, row_vec, vocab, s);
        e = hipGetLastError();
    } else {
        const dim3 grid((unsigned)tokens), block(kBlock);
        const int unit = copy_unit(row_bytes, out, table);
        if (unit == 4)
            hipLaunchKernelGGL(gather_rows_units<uint32_t>, grid, block, 0, s, ids, static_cast<uint32_t*>(out),
                               static_cast<const uint32_t*>(table), tokens, row_bytes / 4, vocab);
        else if (unit == 2)
            hipLaunchKernelGGL(gather_rows_units<uint16_t>, grid, block, 0, s, ids, static_cast<uint16_t*>(out),
                               static_cast<const uint16_t*>(table), tokens, row_bytes / 2, vocab);
        else
            hipLaunchKernelGGL(gather_rows_units<uint8_t>, grid, block, 0, s, ids, static_cast<uint8_t*>(out),
                               static_cast<const uint8_t*>(table), tokens, row_bytes, vocab);
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
