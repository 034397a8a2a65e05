// The strided copies either side of attention, for gfx950: transpose-out + remove padding, KV-cache
// append, KV-cache broadcast.  All three move whole head rows (head_size elements), so they are
// written once on bytes and serve every element type bit-exactly.
//
//   transpose_remove_padding   [batch, heads, seq, hs] -> [tokens, heads, hs]
//       contract: src/kernels/fused_transpose_and_remv_pad.h:7-10 and
//       tests/unittests/test_fused_trans_remv_pad.cu:3,28-49 (the reference declares and tests this
//       launcher but holds no definition); it is the inverse of the QKV scatter
//       (src/kernels/qkv_bias_and_RoPE.cu:135-140).
//   concat_kv_cache            src/kernels/concat_past_kv.cu:7-113
//   repeat_kv_cache            src/kernels/repeat_kv.cu:10-100
//
// Design: one 16-byte vector per lane, a workgroup covers one 4 KiB chunk of the contiguous side,
// non-temporal write-through stores; k and v go in one launch (the reference issues two).  Rows whose index
// would fall outside the destination are skipped instead of written out of bounds.
#include "isp_common.h"

namespace isp {

// Vectors per head row: almost always a power of two (16 for 128 fp16 elements), so the row / column
// split of a flat vector index is a shift and a mask; any other width takes the division.
struct SegSplit {
    unsigned seg_vec;
    int shift;  // log2(seg_vec) or -1
    __device__ __forceinline__ void split(unsigned vi, unsigned& row, unsigned& col) const {
        if (shift >= 0) {
            row = vi >> shift;
            col = vi & (seg_vec - 1u);
        } else {
            row = vi / seg_vec;
            col = vi - row * seg_vec;
        }
    }
};

static SegSplit make_split(unsigned seg_vec) {
    SegSplit sp;
    sp.seg_vec = seg_vec;
    sp.shift = -1;
    if (seg_vec != 0 && (seg_vec & (seg_vec - 1u)) == 0) {
        sp.shift = 0;
        while ((1u << sp.shift) < seg_vec) sp.shift++;
    }
    return sp;
}

// dst[token, h, :] = src[b, h, s, :],  token + padding_offset[token] = b * seq_len + s.
// grid = tokens * chunks, a chunk being BLOCK vectors of the token's heads*seg_vec vectors
template <int BLOCK>
__global__ __launch_bounds__(BLOCK) void transpose_remove_padding_vec(
    const char* __restrict__ src, const int32_t* __restrict__ padding_offset, char* __restrict__ dst,
    unsigned positions, int head_num, FastDiv seq, SegSplit sp, FastDiv chunks) {
    const unsigned seg_vec = sp.seg_vec;
    const unsigned seq_len = seq.d;
    unsigned token, chunk;
    chunks.divmod(blockIdx.x, token, chunk);
    const unsigned vi = chunk * BLOCK + threadIdx.x;  // vector index inside the token's row
    const unsigned row_vec = (unsigned)head_num * seg_vec;
    if (vi >= row_vec) return;
    const long long p = (long long)token + (long long)read_only_i32(padding_offset, (int)token);
    if (p < 0 || p >= (long long)positions) return;
    unsigned b, s;
    seq.divmod((unsigned)p, b, s);
    unsigned h, c;
    sp.split(vi, h, c);
    const size_t from = ((((size_t)b * head_num + h) * seq_len + s) * seg_vec + c) * 16u;
    store16_through(dst + ((size_t)token * row_vec + vi) * 16u, load16_stream(src + from));
}

// Fallbacks for head rows that are not whole aligned 16-byte vectors: copies in units of U (4, 2 or 1
// bytes, the widest the sizes and addresses allow); `seg` counts units per head row.
template <typename U>
__global__ __launch_bounds__(kBlock) void transpose_remove_padding_units(
    const U* src, const int32_t* padding_offset, U* dst, int batch, int head_num, int seq_len,
    size_t seg) {
    const unsigned token = blockIdx.x;
    const long long p = (long long)token + (long long)padding_offset[token];
    if (p < 0 || p >= (long long)batch * seq_len) return;
    const size_t b = (size_t)(p / seq_len), s = (size_t)(p % seq_len);
    const size_t row = (size_t)head_num * seg;
    for (size_t i = threadIdx.x; i < row; i += kBlock) {
        const size_t h = i / seg, c = i % seg;
        dst[(size_t)token * row + i] = src[((b * head_num + h) * seq_len + s) * seg + c];
    }
}

// The grid of the two cache movers below: one workgroup per chunk of BLOCK vectors of every (sequence, head)
// row, k / v in blockIdx.z.  The valid lengths live on the device, so the grid has to cover the maximum
// length of every row, and the workgroups behind a sequence's end leave at once.  Which chunk a workgroup
// takes matters more than how many leave: with chunk = blockIdx.x % chunks the live and the idle
// workgroups repeat with the period of a row, workgroups are handed to the chip's partitions in turn, and
// for row lengths that are multiples of the partition count (32 chunks here) some partitions then receive
// mostly idle ones (batch 8 x 32 heads x 512 positions, every sequence 256 long: 16.1 us; lengths 256..512:
// 18.7 us).  Rotating the chunk index by 5 per row breaks the lockstep: 12.5 and 16.9 us (copies of the same
// bytes: 11.9 and 16.4 us); full rows are unchanged (22.5 us).  Measured and not kept: the rows as the fastest
// grid dimension (24.9 us on full rows: neighbouring workgroups then sit 128 KiB apart), two or four
// interleaved chunks per workgroup (23.5 / 25.1 us on full rows), workgroups of 512 and 1024 threads
// (19.0 / 19.6 us where 256 threads take 18.5 us).
struct MoverGrid {
    FastDiv chunks;  // chunks per row
    __device__ __forceinline__ void locate(unsigned& row, unsigned& chunk) const {
        unsigned j, q, turn;
        chunks.divmod(blockIdx.x, row, j);
        chunks.divmod(row, q, turn);
        chunks.divmod(j + turn * 5u, q, chunk);  // chunks <= 2^23 (a row has at most 2^31 vectors)
    }
};

// cache[b, h, history[b] + t, :] = src[b, h, t, :] for t < cur_len[b]
template <int BLOCK>
__global__ __launch_bounds__(BLOCK) void concat_kv_vec(
    const char* __restrict__ k_src, const char* __restrict__ v_src, char* __restrict__ k_cache,
    char* __restrict__ v_cache, const int32_t* __restrict__ cur_query_length,
    const int32_t* __restrict__ history_length, FastDiv kv_heads, int max_q_len, int max_seq_len,
    SegSplit sp, MoverGrid mg) {
    const unsigned seg_vec = sp.seg_vec;
    const char* src = blockIdx.z == 0 ? k_src : v_src;
    char* cache = blockIdx.z == 0 ? k_cache : v_cache;
    unsigned bh, chunk;
    mg.locate(bh, chunk);
    unsigned b, head;
    kv_heads.divmod(bh, b, head);
    const unsigned vi = chunk * BLOCK + threadIdx.x;
    if (vi >= (unsigned)max_q_len * seg_vec) return;
    unsigned t, c;
    sp.split(vi, t, c);
    const int cur = read_only_i32(cur_query_length, (int)b);
    const long long row = (long long)read_only_i32(history_length, (int)b) + t;
    if ((int)t >= cur || row < 0 || row >= max_seq_len) return;
    store16_through(cache + (((size_t)bh * max_seq_len + (size_t)row) * seg_vec + c) * 16u,
                   load16_stream(src + ((size_t)bh * max_q_len * seg_vec + vi) * 16u));
}

template <typename U>
__global__ __launch_bounds__(kBlock) void concat_kv_units(
    const U* k_src, const U* v_src, U* k_cache, U* v_cache,
    const int32_t* cur_query_length, const int32_t* history_length, int kv_head_num, int max_q_len,
    int max_seq_len, size_t seg) {
    const U* src = blockIdx.z == 0 ? k_src : v_src;
    U* cache = blockIdx.z == 0 ? k_cache : v_cache;
    const unsigned bh = blockIdx.y, b = bh / kv_head_num, t = blockIdx.x;
    const long long row = (long long)history_length[b] + t;
    if ((int)t >= cur_query_length[b] || row < 0 || row >= max_seq_len) return;
    for (size_t i = threadIdx.x; i < seg; i += kBlock)
        cache[((size_t)bh * max_seq_len + (size_t)row) * seg + i] =
            src[((size_t)bh * max_q_len + t) * seg + i];
}

// dst[b, h, s, :] = cache[b, h / rep, s, :] for s < context_length[b]
template <int BLOCK>
__global__ __launch_bounds__(BLOCK) void repeat_kv_vec(
    const char* __restrict__ k_cache, const char* __restrict__ v_cache, char* __restrict__ k_dst,
    char* __restrict__ v_dst, const int32_t* __restrict__ context_length, FastDiv heads, FastDiv group,
    int kv_head_num, int max_seq_len, int max_k_len, SegSplit sp, MoverGrid mg) {
    const unsigned seg_vec = sp.seg_vec;
    const char* cache = blockIdx.z == 0 ? k_cache : v_cache;
    char* dst = blockIdx.z == 0 ? k_dst : v_dst;
    unsigned bh, chunk;
    mg.locate(bh, chunk);
    unsigned b, h;
    heads.divmod(bh, b, h);
    const unsigned vi = chunk * BLOCK + threadIdx.x;
    if (vi >= (unsigned)max_k_len * seg_vec) return;
    unsigned s, c;
    sp.split(vi, s, c);
    if ((int)s >= read_only_i32(context_length, (int)b) || (int)s >= max_seq_len) return;
    unsigned kvh, within;
    group.divmod(h, kvh, within);
    store16_through(dst + ((size_t)bh * max_k_len * seg_vec + vi) * 16u,
                   load16_stream(cache + (((size_t)b * kv_head_num + kvh) * max_seq_len * seg_vec + vi) * 16u));
}

template <typename U>
__global__ __launch_bounds__(kBlock) void repeat_kv_units(
    const U* k_cache, const U* v_cache, U* k_dst, U* v_dst,
    const int32_t* context_length, int head_num, int kv_head_num, int max_seq_len, int max_k_len,
    size_t seg) {
    const U* cache = blockIdx.z == 0 ? k_cache : v_cache;
    U* dst = blockIdx.z == 0 ? k_dst : v_dst;
    const unsigned bh = blockIdx.y, b = bh / head_num, h = bh % head_num, s = blockIdx.x;
    if ((int)s >= context_length[b] || (int)s >= max_seq_len) return;
    const unsigned kvh = h / (unsigned)(head_num / kv_head_num);
    for (size_t i = threadIdx.x; i < seg; i += kBlock)
        dst[((size_t)bh * max_k_len + s) * seg + i] =
            cache[(((size_t)b * kv_head_num + kvh) * max_seq_len + s) * seg + i];
}

constexpr long long kMaxGridYZ = 65535;

// Threads per workgroup of the cache movers: 64 ... 1024 (tuning knob, else the measured default).
static int mover_block() {
    const int knob = tuning(ISP_TUNE_MOVER_BLOCK_THREADS);
    return (knob == 64 || knob == 128 || knob == 256 || knob == 512 || knob == 1024) ? knob : 256;
}

static int transpose_remove_padding(const void* src, const int32_t* padding_offset, void* dst,
                                    int batch, int head_num, int seq_len, int head_size,
                                    int token_num, int elem, hipStream_t s) {
    if (batch < 0 || head_num < 0 || seq_len < 0 || head_size < 0 || token_num < 0) return ISP_ERR_BAD_SHAPE;
    if (token_num == 0 || head_num == 0 || head_size == 0) return ISP_OK;
    if (batch == 0 || seq_len == 0) return ISP_ERR_BAD_SHAPE;
    ISP_REQUIRE_PTR(src);
    ISP_REQUIRE_PTR(padding_offset);
    ISP_REQUIRE_PTR(dst);
    const size_t seg = (size_t)head_size * elem;
    const size_t row_vec = (size_t)head_num * (seg / 16);
    // single-wave workgroups: 9.17 us against 9.5-9.6 with 128, 256 or 512 threads at 2977 tokens of 32 heads
    // (the two cache movers, whose grids hold workgroups that leave at once, measured 2-3 % slower that way
    // and keep 256).  The knob of the cache movers overrides.
    const int knob = tuning(ISP_TUNE_MOVER_BLOCK_THREADS);
    const int blk = (knob == 64 || knob == 128 || knob == 256 || knob == 512) ? knob : 64;
    const size_t chunks = (row_vec + blk - 1) / blk;
    // the vector kernel keeps padded positions in 32 bits and divides with a multiply-high
    if (seg % 16 == 0 && aligned16(src) && aligned16(dst) && chunks * (size_t)token_num <= 0x7fffffffull &&
        (unsigned long long)batch * (unsigned long long)seq_len <= 0x7fffffffull) {
        const unsigned seg_vec = (unsigned)(seg / 16);
        dim3 grid((unsigned)(chunks * (size_t)token_num));
#define ISP_LAUNCH_TRANSPOSE(B)                                                                     \
    hipLaunchKernelGGL(transpose_remove_padding_vec<B>, grid, dim3(B), 0, s,                         \
                       static_cast<const char*>(src), padding_offset, static_cast<char*>(dst),       \
                       (unsigned)batch * (unsigned)seq_len, head_num, make_fastdiv((unsigned)seq_len), \
                       make_split(seg_vec), make_fastdiv((unsigned)chunks))
        if (blk == 512) ISP_LAUNCH_TRANSPOSE(512);
        else if (blk == 128) ISP_LAUNCH_TRANSPOSE(128);
        else if (blk == 64) ISP_LAUNCH_TRANSPOSE(64);
        else ISP_LAUNCH_TRANSPOSE(256);
#undef ISP_LAUNCH_TRANSPOSE
    } else {
        const dim3 grid((unsigned)token_num), block(kBlock);
#define ISP_LAUNCH_UNITS(U)                                                                        \
    hipLaunchKernelGGL(transpose_remove_padding_units<U>, grid, block, 0, s,                        \
                       static_cast<const U*>(src), padding_offset, static_cast<U*>(dst), batch,     \
                       head_num, seq_len, seg / sizeof(U))
        const int unit = copy_unit(seg, src, dst);
        if (unit == 4) ISP_LAUNCH_UNITS(uint32_t);
        else if (unit == 2) ISP_LAUNCH_UNITS(uint16_t);
        else ISP_LAUNCH_UNITS(uint8_t);
#undef ISP_LAUNCH_UNITS
    }
    return note_launch(hipGetLastError());
}

static int concat_kv(const void* k_src, const void* v_src, void* k_cache, void* v_cache, int layer,
                     const int32_t* cur_query_length, const int32_t* history_length, int batch,
                     int kv_head_num, int max_q_len, int max_seq_len, int head_size, int elem,
                     hipStream_t s) {
    if (batch < 0 || kv_head_num < 0 || max_q_len < 0 || max_seq_len < 0 || head_size < 0 || layer < 0)
        return ISP_ERR_BAD_SHAPE;
    if (batch == 0 || kv_head_num == 0 || max_q_len == 0 || head_size == 0) return ISP_OK;
    ISP_REQUIRE_PTR(k_src);
    ISP_REQUIRE_PTR(v_src);
    ISP_REQUIRE_PTR(k_cache);
    ISP_REQUIRE_PTR(v_cache);
    ISP_REQUIRE_PTR(cur_query_length);
    ISP_REQUIRE_PTR(history_length);
    const size_t seg = (size_t)head_size * elem;
    // layer offset = layer * batch * kv_head_num * max_seq_len * head_size elements (concat_past_kv.cu:89)
    const size_t layer_bytes = (size_t)layer * batch * kv_head_num * max_seq_len * seg;
    char* kc = static_cast<char*>(k_cache) + layer_bytes;
    char* vc = static_cast<char*>(v_cache) + layer_bytes;
    const char* ks = static_cast<const char*>(k_src);
    const char* vs = static_cast<const char*>(v_src);
    if (seg % 16 == 0 && aligned16(ks) && aligned16(vs) && aligned16(kc) && aligned16(vc)) {
        const unsigned seg_vec = (unsigned)(seg / 16);
        const size_t row_vec = (size_t)max_q_len * seg_vec;
        if (row_vec > 0x7fffffffull) return ISP_ERR_UNSUPPORTED;  // 32-bit vector indices, with room for the last workgroup
        const int blk = mover_block();
        const size_t chunks = (row_vec + blk - 1) / blk;
        if (chunks * (size_t)batch * kv_head_num > 0x7fffffffull) return ISP_ERR_UNSUPPORTED;
        const dim3 grid((unsigned)(chunks * (size_t)batch * kv_head_num), 1, 2);
        const MoverGrid mg{make_fastdiv((unsigned)chunks)};
#define ISP_LAUNCH_CONCAT(B)                                                                       \
    hipLaunchKernelGGL(concat_kv_vec<B>, grid, dim3(B), 0, s, ks, vs, kc, vc, cur_query_length,     \
                       history_length, make_fastdiv((unsigned)kv_head_num), max_q_len, max_seq_len,       \
                       make_split(seg_vec), mg)
        if (blk == 1024) ISP_LAUNCH_CONCAT(1024);
        else if (blk == 512) ISP_LAUNCH_CONCAT(512);
        else if (blk == 128) ISP_LAUNCH_CONCAT(128);
        else if (blk == 64) ISP_LAUNCH_CONCAT(64);
        else ISP_LAUNCH_CONCAT(256);
#undef ISP_LAUNCH_CONCAT
    } else {
        if ((long long)batch * kv_head_num > kMaxGridYZ) return ISP_ERR_UNSUPPORTED;
        const dim3 grid((unsigned)max_q_len, (unsigned)(batch * kv_head_num), 2), block(kBlock);
#define ISP_LAUNCH_UNITS(U)                                                                        \
    hipLaunchKernelGGL(concat_kv_units<U>, grid, block, 0, s, reinterpret_cast<const U*>(ks),       \
                       reinterpret_cast<const U*>(vs), reinterpret_cast<U*>(kc),                    \
                       reinterpret_cast<U*>(vc), cur_query_length, history_length, kv_head_num,     \
                       max_q_len, max_seq_len, seg / sizeof(U))
        const int unit = copy_unit(seg, ks, vs, kc, vc);
        if (unit == 4) ISP_LAUNCH_UNITS(uint32_t);
        else if (unit == 2) ISP_LAUNCH_UNITS(uint16_t);
        else ISP_LAUNCH_UNITS(uint8_t);
#undef ISP_LAUNCH_UNITS
    }
    return note_launch(hipGetLastError());
}

static int repeat_kv(const void* k_cache, const void* v_cache, void* k_dst, void* v_dst, int layer,
                     const int32_t* context_length, int batch, int head_num, int kv_head_num,
                     int max_seq_len, int max_k_len, int head_size, int elem, hipStream_t s) {
    if (batch < 0 || head_num < 0 || kv_head_num < 0 || max_seq_len < 0 || max_k_len < 0 ||
        head_size < 0 || layer < 0)
        return ISP_ERR_BAD_SHAPE;
    if (batch == 0 || head_num == 0 || max_k_len == 0 || head_size == 0) return ISP_OK;
    if (kv_head_num == 0 || head_num % kv_head_num != 0) return ISP_ERR_BAD_SHAPE;
    ISP_REQUIRE_PTR(k_cache);
    ISP_REQUIRE_PTR(v_cache);
    ISP_REQUIRE_PTR(k_dst);
    ISP_REQUIRE_PTR(v_dst);
    ISP_REQUIRE_PTR(context_length);
    const size_t seg = (size_t)head_size * elem;
    const size_t layer_bytes = (size_t)layer * batch * kv_head_num * max_seq_len * seg;  // repeat_kv.cu:70
    const char* kc = static_cast<const char*>(k_cache) + layer_bytes;
    const char* vc = static_cast<const char*>(v_cache) + layer_bytes;
    char* kd = static_cast<char*>(k_dst);
    char* vd = static_cast<char*>(v_dst);
    if (seg % 16 == 0 && aligned16(kc) && aligned16(vc) && aligned16(kd) && aligned16(vd)) {
        const unsigned seg_vec = (unsigned)(seg / 16);
        const size_t row_vec = (size_t)max_k_len * seg_vec;
        if (row_vec > 0x7fffffffull) return ISP_ERR_UNSUPPORTED;  // 32-bit vector indices, with room for the last workgroup
        const int blk = mover_block();
        const size_t chunks = (row_vec + blk - 1) / blk;
        if (chunks * (size_t)batch * head_num > 0x7fffffffull) return ISP_ERR_UNSUPPORTED;
        const dim3 grid((unsigned)(chunks * (size_t)batch * head_num), 1, 2);
        const MoverGrid mg{make_fastdiv((unsigned)chunks)};
#define ISP_LAUNCH_REPEAT(B)                                                                       \
    hipLaunchKernelGGL(repeat_kv_vec<B>, grid, dim3(B), 0, s, kc, vc, kd, vd, context_length,       \
                       make_fastdiv((unsigned)head_num), make_fastdiv((unsigned)(head_num / kv_head_num)),    \
                       kv_head_num, max_seq_len, max_k_len, make_split(seg_vec), mg)
        if (blk == 1024) ISP_LAUNCH_REPEAT(1024);
        else if (blk == 512) ISP_LAUNCH_REPEAT(512);
        else if (blk == 128) ISP_LAUNCH_REPEAT(128);
        else if (blk == 64) ISP_LAUNCH_REPEAT(64);
        else ISP_LAUNCH_REPEAT(256);
#undef ISP_LAUNCH_REPEAT
    } else {
        if ((long long)batch * head_num > kMaxGridYZ) return ISP_ERR_UNSUPPORTED;
        const dim3 grid((unsigned)max_k_len, (unsigned)(batch * head_num), 2), block(kBlock);
#define ISP_LAUNCH_UNITS(U)                                                                        \
    hipLaunchKernelGGL(repeat_kv_units<U>, grid, block, 0, s, reinterpret_cast<const U*>(kc),       \
                       reinterpret_cast<const U*>(vc), reinterpret_cast<U*>(kd),                    \
                       reinterpret_cast<U*>(vd), context_length, head_num, kv_head_num,             \
                       max_seq_len, max_k_len, seg / sizeof(U))
        const int unit = copy_unit(seg, kc, vc, kd, vd);
        if (unit == 4) ISP_LAUNCH_UNITS(uint32_t);
        else if (unit == 2) ISP_LAUNCH_UNITS(uint16_t);
        else ISP_LAUNCH_UNITS(uint8_t);
#undef ISP_LAUNCH_UNITS
    }
    return note_launch(hipGetLastError());
}

}  // namespace isp

extern "C" {

int isp_transpose_remove_padding_f32(const void* src, const int32_t* padding_offset, void* dst,
                                     int batch, int head_num, int seq_len, int head_size,
                                     int token_num, isp_stream_t stream) {
    return isp::transpose_remove_padding(src, padding_offset, dst, batch, head_num, seq_len, head_size,
                                         token_num, 4, static_cast<hipStream_t>(stream));
}
int isp_transpose_remove_padding_f16(const void* src, const int32_t* padding_offset, void* dst,
                                     int batch, int head_num, int seq_len, int head_size,
                                     int token_num, isp_stream_t stream) {
    return isp::transpose_remove_padding(src, padding_offset, dst, batch, head_num, seq_len, head_size,
                                         token_num, 2, static_cast<hipStream_t>(stream));
}

int isp_concat_kv_cache_f32(const void* k_src, const void* v_src, void* k_cache, void* v_cache,
                            int layer, const int32_t* cur_query_length,
                            const int32_t* history_length, int batch, int kv_head_num, int max_q_len,
                            int max_seq_len, int head_size, isp_stream_t stream) {
    return isp::concat_kv(k_src, v_src, k_cache, v_cache, layer, cur_query_length, history_length,
                          batch, kv_head_num, max_q_len, max_seq_len, head_size, 4,
                          static_cast<hipStream_t>(stream));
}
int isp_concat_kv_cache_f16(const void* k_src, const void* v_src, void* k_cache, void* v_cache,
                            int layer, const int32_t* cur_query_length,
                            const int32_t* history_length, int batch, int kv_head_num, int max_q_len,
                            int max_seq_len, int head_size, isp_stream_t stream) {
    return isp::concat_kv(k_src, v_src, k_cache, v_cache, layer, cur_query_length, history_length,
                          batch, kv_head_num, max_q_len, max_seq_len, head_size, 2,
                          static_cast<hipStream_t>(stream));
}

int isp_repeat_kv_cache_f32(const void* k_cache, const void* v_cache, void* k_dst, void* v_dst,
                            int layer, const int32_t* context_length, int batch, int head_num,
                            int kv_head_num, int max_seq_len, int max_k_len, int head_size,
                            isp_stream_t stream) {
    return isp::repeat_kv(k_cache, v_cache, k_dst, v_dst, layer, context_length, batch, head_num,
                          kv_head_num, max_seq_len, max_k_len, head_size, 4,
                          static_cast<hipStream_t>(stream));
}
int isp_repeat_kv_cache_f16(const void* k_cache, const void* v_cache, void* k_dst, void* v_dst,
                            int layer, const int32_t* context_length, int batch, int head_num,
                            int kv_head_num, int max_seq_len, int max_k_len, int head_size,
                            isp_stream_t stream) {
    return isp::repeat_kv(k_cache, v_cache, k_dst, v_dst, layer, context_length, batch, head_num,
                          kv_head_num, max_seq_len, max_k_len, head_size, 2,
                          static_cast<hipStream_t>(stream));
}

}  // extern "C"
