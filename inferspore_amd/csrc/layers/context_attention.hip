// Fused causal attention of the context-decoder layer for fp16 heads of 128 or 64 elements: one kernel in place of
// KV broadcast, q x k^T, masked softmax, p x v and the transpose back to packed tokens.  It reads the padded
// queries [batch, head_num, max_q_len, hs], the layer's slice of the KV cache [batch, kv_head_num,
// max_seq_len, hs] (keys and values of the history and of this call's tokens) and writes the packed
// [tokens, head_num, hs] rows the output projection consumes.  The [queries x keys] scores never leave the
// registers, and key tiles behind the causal diagonal are not visited.
//
// The mask is the one of the layer's softmax: query q of sequence b sees the keys at positions
// < min(history_length[b] + q + 1, context_length[b], max_k_len).  A deliberate departure from the reference when a
// sequence has history: its mask (src/kernels/build_casual_mask.cu:36) additionally requires k >= context length -
// query length, which hides every history key -- the comment above that line calls it the mask that does not support
// multi-turn dialogue and draws the one that does, which is the one computed here.  With history_length = 0 the two
// are the same mask.
//
// Matrix cores: v_mfma_f32_32x32x16_f16.  A wavefront owns 32 queries.  It computes the TRANSPOSED scores
// S^T[key, query] = K x Q^T, so that a lane's 16 accumulators of a 32 x 32 block all belong to one query
// (column = lane % 32): the running maximum and sum of the online softmax are per-lane scalars, combined only
// with the other half of the wavefront (lane ^ 32), and the probabilities are, as they sit in the
// accumulators, the B operand of the second product O^T[d, query] = V^T x P^T -- no exchange between lanes.
// The B operand's 16 contraction indices are matched to the accumulator rows by reading V^T's keys in the
// order (4 h + j, 8 + 4 h + j), h = lane / 32: a contraction does not care about the order of its terms as
// long as both operands agree.  K tiles sit in LDS as stored ([key][d], padded rows), V tiles transposed
// ([d][key], written two keys at a time, the keys of a row in the operand's order) so that the A operand of the
// second product is one 16-byte read.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <string>

#include "src/layers/decoder/context_decoder_layer.h"
#include "src/utils/macro.h"

namespace isp_layers {

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kQueriesPerWave = 32;
constexpr int kWaves = 4;
constexpr int kQueryTile = kQueriesPerWave * kWaves;  // queries per workgroup
constexpr int kKeyTile = 64;
constexpr int kKPad = 8;  // halfs added to a key row in LDS (272 bytes for 128-element heads): spreads the rows over the banks

// The transposed value tile: row d holds the tile's 64 keys as 8 units of 16 bytes, and a unit is exactly what one
// lane needs for one product: unit 2 t + h holds the keys 16 t + 4 h + 0..3 followed by 16 t + 8 + 4 h + 0..3 (the
// order in which the accumulator rows of the scores meet the operand's contraction index).  Unit u of row d sits
// at position u ^ (d % 8) ^ ((d / 8) % 8): the 64 lanes of an operand read (32 rows d, two units) then touch every
// bank equally, and the transposing writes (two neighbouring keys, 4 bytes) are spread over half of the banks.
__device__ __forceinline__ int vt_unit(int d, int unit) { return d * (kKeyTile / 2) + 4 * (unit ^ (d & 7) ^ ((d >> 3) & 7)); }
// dword that holds the keys `pair * 2` and `pair * 2 + 1` of row d
__device__ __forceinline__ int vt_pair(int d, int pair) {
    const int key = 2 * pair, step = key / 16, quad = (key % 16) / 4;  // quads 0..3 of a step: h = quad % 2, second half = quad / 2
    return vt_unit(d, 2 * step + quad % 2) + 2 * (quad / 2) + (key % 4) / 2;
}

__device__ __forceinline__ int uniform_int(const int* p, int i) {
    // the lengths never change while the kernel runs: read them through the scalar cache
    typedef const int __attribute__((address_space(4)))* constant_ints;
    return reinterpret_cast<constant_ints>((unsigned long long)p)[i];
}

// Maximum / sum of a value with the one in the other half of the wavefront (lane ^ 32), without a trip through LDS:
// the swap leaves the lower half's value in every lane of one register and the upper half's in the other.
__device__ __forceinline__ float halves_max(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float halves_sum(float x) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <int HS>  // head size: 128 or 64
__global__ __launch_bounds__(256, 2) void context_attention_f16(
    const _Float16* __restrict__ q_buf, const _Float16* __restrict__ k_cache, const _Float16* __restrict__ v_cache,
    _Float16* __restrict__ out, const int* history_length, const int* input_length, const int* context_length,
    int head_num, int kv_head_num, int max_q_len, int max_k_len, int max_seq_len, int tokens, float scale_log2e) {
    constexpr int kHeadSize = HS, kKStride = HS + kKPad;
    constexpr int kDSteps = HS / 16;    // products over d per 32 x 32 block of scores
    constexpr int kDBlocks = HS / 32;   // 32-row blocks of O^T
    constexpr int kChunks = HS / 8;     // 16-byte pieces of a key or value row
    constexpr int kMoves = HS / 64;     // key pairs a thread moves per tile
    __shared__ __align__(16) _Float16 k_tiles[2][kKeyTile * kKStride];
    __shared__ __align__(16) uint32_t vt_tiles[2][kHeadSize * kKeyTile / 2];  // [d][key], two keys per dword

    const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64, half_id = lane / 32, col = lane % 32;
    // grid: x = head (fastest), y = sequence, z = query tile in DESCENDING order -- the tiles far down the causal
    // triangle visit the most key tiles, and workgroups are handed out in grid order, so the long ones start first
    // (the kernel takes as long as its longest workgroup: pinning the query tiles of a (sequence, head) pair to one
    // XCD so that they share its L2 gives up that order and measured 50 instead of 41 us)
    const int head = blockIdx.x, b = blockIdx.y, q0 = (int)(gridDim.z - 1 - blockIdx.z) * kQueryTile;
    const int len = min(uniform_int(input_length, b), max_q_len);
    if (q0 >= len) return;  // workgroup-uniform: only padded queries here
    const int hist = uniform_int(history_length, b);
    const int ctx = min(min(uniform_int(context_length, b), max_k_len), max_seq_len);
    int first_token = 0;
    for (int i = 0; i < b; i++) first_token += uniform_int(input_length, i);
    const int kv_head = head / (head_num / kv_head_num);
    const size_t kv_offset = ((size_t)b * kv_head_num + kv_head) * (size_t)max_seq_len * kHeadSize;
    const _Float16* keys = k_cache + kv_offset;
    const _Float16* values = v_cache + kv_offset;

    // keys the workgroup's last real query sees, the wavefront's last real query, this lane's query
    const int wg_visible = min(hist + min(q0 + kQueryTile, len), ctx);
    const int wave_q0 = q0 + wave * kQueriesPerWave;
    const int wave_visible = wave_q0 < len ? min(hist + min(wave_q0 + kQueriesPerWave, len), ctx) : 0;
    // keys that every query of the wavefront sees: its first query's, or none if the wavefront has padded lanes
    const int wave_all_visible = wave_q0 + kQueriesPerWave <= len ? min(hist + wave_q0 + 1, ctx) : 0;
    const int my_q = wave_q0 + col;
    const bool real = my_q < len;
    const int my_visible = real ? min(hist + my_q + 1, ctx) : 0;

    const long long token = (long long)first_token + my_q;
    if (wg_visible <= 0) {  // workgroup-uniform: a context of no keys (inconsistent lengths); nothing to attend to
        if (real && token < tokens) {
            _Float16* o_row = out + ((size_t)token * head_num + head) * kHeadSize;
            for (int d = 8 * half_id; d < kHeadSize; d += 16) *reinterpret_cast<uint4*>(o_row + d) = make_uint4(0u, 0u, 0u, 0u);
        }
        return;
    }

    // Q^T as the B operand: lane (col, half_id) holds q[my_q][16 s + 8 half_id + 0..7] for the 8 steps over d
    half8 qf[kDSteps];
    {
        const _Float16* q_row = q_buf + (((size_t)b * head_num + head) * (size_t)max_q_len + (size_t)(real ? my_q : q0)) * kHeadSize;
#pragma unroll
        for (int s = 0; s < kDSteps; s++) {
            qf[s] = *reinterpret_cast<const half8*>(q_row + 16 * s + 8 * half_id);
            if (!real) qf[s] = half8{0, 0, 0, 0, 0, 0, 0, 0};
        }
    }

    float16v acc[kDBlocks];  // O^T[d = 32 db + rows, query = col]
#pragma unroll
    for (int db = 0; db < kDBlocks; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[db][i] = 0.0f;
    float run_max = -INFINITY, run_sum = 0.0f;

    // A thread moves two pairs of neighbouring keys per tile (pairs, so that V^T is written two keys -- one dword --
    // at a time).  The eight loads of a tile are issued together and unconditionally: a row past the visible keys
    // re-reads the last visible one and is masked to zero when it is stored (loads or register writes under a
    // branch would each be waited for before the next is issued).  The loads of tile n + 1 are in flight while
    // tile n is computed.
    uint4 kraw[kMoves][2], vraw[kMoves][2];
    auto fetch = [&](int kt) {
#pragma unroll
        for (int i = 0; i < kMoves; i++) {
            const int unit = tid + 256 * i, d0 = (unit % kChunks) * 8, key = 2 * (unit / kChunks);
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const size_t at = (size_t)min(kt + key + j, wg_visible - 1) * kHeadSize + d0;
                kraw[i][j] = *reinterpret_cast<const uint4*>(keys + at);
                vraw[i][j] = *reinterpret_cast<const uint4*>(values + at);
            }
        }
    };
    auto store = [&](int buf, int kt) {
        _Float16* k_lds = k_tiles[buf];
        uint32_t* vt_lds = vt_tiles[buf];
        // ---- the tile into LDS: 64 keys x 128 d of K as stored, of V transposed; keys past the visible ones as zeros
        //      (a zero probability times whatever an unwritten cache row holds could be NaN)
#pragma unroll
        for (int i = 0; i < kMoves; i++) {
            const int unit = tid + 256 * i, pair = unit / kChunks, d0 = (unit % kChunks) * 8, key = 2 * pair;
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int j = 0; j < 2; j++) {
                uint4 kk = kraw[i][j], vv = vraw[i][j];
                if (kt + kKeyTile > wg_visible) {  // workgroup-uniform: only the last tile has rows to blank
                    const uint32_t keep = kt + key + j < wg_visible ? 0xffffffffu : 0u;
                    kk = make_uint4(kk.x & keep, kk.y & keep, kk.z & keep, kk.w & keep);
                    vv = make_uint4(vv.x & keep, vv.y & keep, vv.z & keep, vv.w & keep);
                }
                *reinterpret_cast<uint4*>(&k_lds[(key + j) * kKStride + d0]) = kk;
                uint32_t* v = j == 0 ? lo : hi;
                v[0] = vv.x, v[1] = vv.y, v[2] = vv.z, v[3] = vv.w;
            }
#pragma unroll
            for (int e = 0; e < 8; e++) {
                // low half: v[key][d0 + e], high half: v[key + 1][d0 + e]  (one byte-permute of the two source dwords)
                vt_lds[vt_pair(d0 + e, pair)] =
                    __builtin_amdgcn_perm(hi[e / 2], lo[e / 2], e % 2 ? 0x07060302u : 0x05040100u);
            }
        }
    };
    fetch(0);
    store(0, 0);
    fetch(kKeyTile);  // past the last tile a fetch re-reads the last visible row; what it brings is stored as zeros
    __syncthreads();

    int cur = 0;
    for (int kt = 0; kt < wg_visible; kt += kKeyTile, cur ^= 1) {
        const _Float16* k_lds = k_tiles[cur];
        const uint32_t* vt_lds = vt_tiles[cur];

        if (kt < wave_visible) {  // wavefront-uniform: tiles behind this wavefront's diagonal are skipped
            // ---- S^T[key, query] for the 64 keys: two 32-row blocks, 8 steps over d each
            // The operand reads of a block are issued together, ahead of the products that use them: read one at a
            // time, each would be waited for (an LDS round trip of a hundred cycles and more) before its product.
            float16v s[2];
#pragma unroll
            for (int rb = 0; rb < 2; rb++) {
#pragma unroll
                for (int i = 0; i < 16; i++) s[rb][i] = 0.0f;
                half8 ka[kDSteps];
#pragma unroll
                for (int st = 0; st < kDSteps; st++)
                    ka[st] = *reinterpret_cast<const half8*>(&k_lds[(32 * rb + col) * kKStride + 16 * st + 8 * half_id]);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int st = 0; st < kDSteps; st++) s[rb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ka[st], qf[st], s[rb], 0, 0, 0);
            }
            // ---- online softmax; accumulator i of block rb is key kt + 32 rb + 8 (i / 4) + 4 half_id + i % 4
            float tile_max = -INFINITY;
            if (kt + kKeyTile > wave_all_visible) {  // wavefront-uniform: some query of this wavefront does not see the whole tile
#pragma unroll
                for (int rb = 0; rb < 2; rb++)
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int key = kt + 32 * rb + 8 * (i / 4) + 4 * half_id + (i % 4);
                        s[rb][i] = key < my_visible ? s[rb][i] : -INFINITY;
                    }
            }
#pragma unroll
            for (int rb = 0; rb < 2; rb++)
#pragma unroll
                for (int i = 0; i < 16; i++) tile_max = fmaxf(tile_max, s[rb][i]);
            tile_max = halves_max(tile_max);
            const float new_max = fmaxf(run_max, tile_max);
            const float safe_max = new_max == -INFINITY ? 0.0f : new_max;  // a query with no visible key yet
            const float rescale = __builtin_amdgcn_exp2f((run_max - safe_max) * scale_log2e);
            const float mc = safe_max * scale_log2e;
            float tile_sum = 0.0f;
#pragma unroll
            for (int rb = 0; rb < 2; rb++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    s[rb][i] = __builtin_amdgcn_exp2f(fmaf(s[rb][i], scale_log2e, -mc));
                    tile_sum += s[rb][i];
                }
            tile_sum = halves_sum(tile_sum);
            run_sum = run_sum * rescale + tile_sum;
            run_max = new_max;
            if (__any(rescale != 1.0f)) {  // the running maximum moves in the first tiles and rarely afterwards
#pragma unroll
                for (int db = 0; db < kDBlocks; db++)
#pragma unroll
                    for (int i = 0; i < 16; i++) acc[db][i] *= rescale;
            }
            // ---- O^T += V^T x P^T, 16 keys per step
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int rb = t / 2, g0 = 2 * (t % 2);
                half8 va[kDBlocks];
#pragma unroll
                for (int db = 0; db < kDBlocks; db++)
                    va[db] = *reinterpret_cast<const half8*>(&vt_lds[vt_unit(32 * db + col, 2 * t + half_id)]);
                half8 p;
#pragma unroll
                for (int e = 0; e < 8; e++) p[e] = (_Float16)s[rb][4 * (g0 + e / 4) + (e % 4)];
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int db = 0; db < kDBlocks; db++) acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[db], p, acc[db], 0, 0, 0);
            }
        }
        // the next tile (its loads were issued before this tile's products) goes into the other buffer, which every
        // wavefront finished reading before the barrier that ended the previous iteration; then the loads of the
        // tile after it are started: one barrier per tile, and no load is waited for right after it was issued
        store(cur ^ 1, kt + kKeyTile);
        fetch(kt + 2 * kKeyTile);
        __syncthreads();
    }

    // ---- O^T / sum -> the packed token row; accumulator i of block db is d = 32 db + 8 (i / 4) + 4 half_id + i % 4
    if (real && token < tokens) {
        const float inv = run_sum > 0.0f ? 1.0f / run_sum : 0.0f;
        _Float16* o_row = out + ((size_t)token * head_num + head) * kHeadSize;
#pragma unroll
        for (int db = 0; db < kDBlocks; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                half4 v;
#pragma unroll
                for (int j = 0; j < 4; j++) v[j] = (_Float16)(acc[db][4 * g + j] * inv);
                *reinterpret_cast<half4*>(o_row + 32 * db + 8 * g + 4 * half_id) = v;
            }
    }
}

}  // namespace

bool fused_context_attention_supports(int head_size, int head_num, int kv_head_num) {
    return (head_size == 128 || head_size == 64) && kv_head_num > 0 && head_num % kv_head_num == 0;
}

void launch_fused_context_attention(const half* q_buf, const half* k_cache, const half* v_cache, half* out,
                                    const int* history_length, const int* input_length, const int* context_length,
                                    int batch, int head_num, int kv_head_num, int head_size, int max_q_len,
                                    int max_k_len, int max_seq_len, int tokens, float scale) {
    LLM_CHECK_WITH_INFO(q_buf && k_cache && v_cache && out && history_length && input_length && context_length,
                        "fused attention: null operand");
    LLM_CHECK_WITH_INFO(head_size == 128 || head_size == 64, "fused attention: heads of 128 or 64 elements only");
    LLM_CHECK_WITH_INFO(batch > 0 && batch <= 65535 && head_num > 0 && kv_head_num > 0 && head_num % kv_head_num == 0 &&
                            max_q_len > 0 && (max_q_len + kQueryTile - 1) / kQueryTile <= 65535 && max_k_len > 0 && max_seq_len > 0 &&
                            tokens >= 0 && scale > 0.0f,
                        "fused attention: extents out of range");
    const uintptr_t bits = reinterpret_cast<uintptr_t>(q_buf) | reinterpret_cast<uintptr_t>(k_cache) |
                           reinterpret_cast<uintptr_t>(v_cache) | reinterpret_cast<uintptr_t>(out);
    LLM_CHECK_WITH_INFO((bits & 15u) == 0, "fused attention: operands must be 16-byte aligned");
    const dim3 grid((unsigned)head_num, (unsigned)batch, (unsigned)((max_q_len + kQueryTile - 1) / kQueryTile));
#define ISP_LAUNCH_ATTENTION(HS)                                                                                  \
    hipLaunchKernelGGL(context_attention_f16<HS>, grid, dim3(256), 0, nullptr,                                    \
                       reinterpret_cast<const _Float16*>(q_buf), reinterpret_cast<const _Float16*>(k_cache),      \
                       reinterpret_cast<const _Float16*>(v_cache), reinterpret_cast<_Float16*>(out), history_length, \
                       input_length, context_length, head_num, kv_head_num, max_q_len, max_k_len, max_seq_len,   \
                       tokens, scale * 1.4426950408889634f)
    if (head_size == 128) ISP_LAUNCH_ATTENTION(128);
    else ISP_LAUNCH_ATTENTION(64);
#undef ISP_LAUNCH_ATTENTION
    CHECK(hipGetLastError());
}

}  // namespace isp_layers
