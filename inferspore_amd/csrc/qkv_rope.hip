// Fused QKV bias + rotate-half RoPE + head transpose + re-padding (prefill) for gfx950.
//
// Semantics: src/kernels/qkv_bias_and_RoPE.cu:132-191 (fp32 kernel) with the bias indexing of that
// file's disabled fp16 body (:239,247,250):
//   p = token + padding_offset[token];  b = p / seq_len;  s = p % seq_len;  t = history[b] + s
//   x = qkv[token, head, d] (+ bias[head, d])
//   q/k heads, d < rot/2:  angle = t / base^(2d/rot)
//       out[d]        = cos * x[d]        - sin * x[d + hs/2]
//       out[d + hs/2] = cos * x[d + hs/2] + sin * x[d]
//   v heads and un-rotated elements are copied;  destination [b, head, s, :] of q / k / v.
//
// Design (not the reference's one-thread-per-element, one-block-per-(token, head) kernel):
//   * the divisors base^(2d/rot) do not depend on the data, so the host computes them once with the
//     C library's powf and passes them by value in the kernel arguments; the device forms
//     angle = t / divisor with one correctly rounded division and evaluates full-range sincosf;
//   * the token's 64 distinct (cos, sin) pairs are evaluated once per workgroup, one pair per lane
//     of its first wave, and handed to the other waves through LDS behind a barrier that they reach
//     while their own loads are in flight (the reference evaluates powf + cos + sin for every
//     (head, d): 48 to 96 times more transcendental work);
//   * the streamed loads are issued before anything that depends on padding_offset / history;
//   * the kernels that share this: qkv_rope_lean_f16 / qkv_rope_lean_f32 for the common LLaMA shape
//     (one 16-byte vector per lane, the rotation partner fetched from another lane in the VALU, scalar
//     address arithmetic), qkv_rope_lean64_f16 for 64-element heads, and qkv_rope_wave for every other
//     vectorisable shape (a lane owns 16 bytes at d = VEC*g and the 16 bytes of its rotation partners
//     at d + hs/2, so the rotate-half pairing needs no cross-lane exchange); all read and write whole
//     128-byte lines of the head rows and give identical bits;
//   * stores are non-temporal write-through (q, k, v are consumed by a later kernel).
#include <math.h>
#include <stddef.h>

#include <type_traits>

#include "isp_common.h"

namespace isp {

constexpr int kMaxHalfRot = 128;  // rotary_embedding_dim up to 256

struct RopeDivisors {
    float div[kMaxHalfRot];
};

// Optional KV-cache append fused into the prefill step (what launchConcatKVCache does afterwards in
// the reference, src/kernels/concat_past_kv.cu:7-73): the k and v rows of a token at position s of
// sequence b also go to cache[b, head, history_length[b] + s, :] when s < input_length[b] and the row
// lies inside the cache.  k_cache / v_cache point at the layer's slice; NULL = no append.
template <typename T>
struct KvAppend {
    T* k_cache;
    T* v_cache;
    const int32_t* input_length;
    int max_seq_len;
};

// Row of the cache a token at (b, s) is appended to, or -1.
template <typename T>
__device__ __forceinline__ long long append_row(const KvAppend<T>& ap, const int32_t* history_length, int b, int s) {
    if (ap.k_cache == nullptr || s >= read_only_i32(ap.input_length, b)) return -1;
    const long long row = (long long)read_only_i32(history_length, b) + s;
    return (row >= 0 && row < ap.max_seq_len) ? row : -1;
}

// (cos, sin) of timestep / divisor: one correctly rounded division and the full-range sincosf, the
// same two operations in every kernel of this file, so a decode step at `step` and a prefill token at
// history = step - 1 produce identical bits (tested).  Inlined on purpose: a device function call
// starts by waiting for all outstanding memory operations, which would put the evaluation behind
// the arrival of the streamed loads instead of underneath it.
__device__ __forceinline__ float2 rope_coefficients(int timestep, float divisor) {
    float sn, c;
    sincosf((float)timestep / divisor, &sn, &c);
    return make_float2(c, sn);
}

// Word `index` of the first kernel argument (the divisor table), read through a plain global pointer
// to the argument block.  Vector-memory results return in issue order; qkv_rope_lean_f16 wants this
// word requested before its streamed row, so that the coefficient evaluation waits for it alone.
// An ordinary argument access would not do: the compiler treats argument loads as movable at will
// and places this one behind the rows'.  The tensors of such a kernel carry no __restrict__ for the
// same reason (their loads must stay where the ordering barriers put them).
__device__ __forceinline__ float first_argument_word(unsigned index) {
    typedef const float __attribute__((address_space(1)))* global_floats;
    unsigned long long block = (unsigned long long)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(block));
    return reinterpret_cast<global_floats>(block)[index];
}

// One rotation, with the contraction spelled out so that every kernel in this file rounds the same
// way: y0 = c x0 - s x1, y1 = c x1 + s x0, each as one product plus one fused multiply-add.
__device__ __forceinline__ void rotate_pair(float c, float sn, float x0, float x1, float& y0,
                                            float& y1) {
    y0 = __fmaf_rn(c, x0, -(sn * x1));
    y1 = __fmaf_rn(c, x1, sn * x0);
}

// A wave owns kWave / G consecutive heads of one token (one head-half pair per lane: two loads and
// two stores).  The first wave of a workgroup evaluates the token's (cos, sin) pairs (lane d
// evaluates pair d) and shares them through LDS behind one barrier (measured 3 % faster than every
// wave evaluating its own copy); workgroups that only carry v heads skip both.
// grid = (tokens, head groups of WAVES waves).
template <typename T, int HS, int ST, int WAVES, bool BIAS>
__global__ __launch_bounds__(kWave * WAVES) void qkv_rope_wave(
    RopeDivisors tab, T* q, T* k, T* v, const T* qkv, const T* bias,
    const int32_t* __restrict__ padding_offset, const int32_t* __restrict__ history_length,
    unsigned positions, FastDiv seq, int head_num, int kv_head_num, int half_rot, KvAppend<T> ap) {
    constexpr int VEC = Elem<T>::kVec;
    constexpr int HALF = HS / 2;
    constexpr int G = HALF / VEC;
    const int seq_len = (int)seq.d;
    static_assert(HALF % VEC == 0 && kWave % G == 0 && HALF <= kWave, "unsupported head size");
    constexpr int HEADS_PER_WAVE = kWave / G;

    // grid = (tokens, head groups): the token index runs fastest, so the workgroups in flight at any
    // time read 8 KiB slices of consecutive token rows and write into one group of 32 heads
    // (measured: faster than token-major order, than 4-token workgroups, and than a layout with
    // one vector per lane and a DPP exchange of the rotation partners).
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int token = (int)blockIdx.x;
    const int g = lane % G;
    const int slot = lane / G;
    const int qkv_heads = head_num + 2 * kv_head_num;
    const int wave_first = ((int)blockIdx.y * WAVES + wave) * HEADS_PER_WAVE;
    const int h = wave_first + slot;
    const bool live = h < qkv_heads;
    const int col = g * VEC;
    const int h_c = live ? h : 0;
    const T* src = qkv + ((size_t)token * (size_t)qkv_heads + h_c) * HS;

    // The source address depends on the token index only, so the streamed loads are issued before
    // the destination (padding_offset -> batch row -> history) is known: the dependent scalar
    // loads then overlap the HBM latency instead of preceding it.  In front of them goes the request
    // for this lane's divisor (see first_argument_word; `tab` MUST stay the first parameter), and every
    // load is unconditional -- lanes without a head read head 0 and discard it, the bias is a template
    // argument -- so that the compiler can count what is outstanding and the first wave's evaluation
    // waits for the divisor alone (with a load inside a branch it waits for everything).
    const float my_divisor = first_argument_word((unsigned)lane);
    (void)tab;
    asm volatile("" ::: "memory");
    const vec16 lo = load16_stream(src + col);
    const vec16 hi = load16_stream(src + HALF + col);
    asm volatile("" ::: "memory");
    vec16 blo, bhi;
    if (BIAS) {
        blo = load16(bias + (size_t)h_c * HS + col);
        bhi = load16(bias + (size_t)h_c * HS + HALF + col);
    }
    asm volatile("" ::: "memory");
    // wave-uniform: scalar arithmetic, the division by seq_len as a multiply-high
    const long long p = (long long)token + (long long)read_only_i32(padding_offset, (int)token);
    if (p < 0 || p >= (long long)positions) return;
    unsigned ub, us;
    seq.divmod((unsigned)p, ub, us);
    const int b = (int)ub, s = (int)us;

    float c[VEC], sn[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) { c[e] = 1.0f; sn[e] = 0.0f; }
    // (cos, sin) of the token: evaluated once per workgroup by its first wave
    const int block_first = (int)blockIdx.y * WAVES * HEADS_PER_WAVE;
    if (block_first < head_num + kv_head_num) {  // workgroup-uniform
        __shared__ float2 cs[HALF];
        if (wave == 0 && lane < HALF) {
            float2 coef = make_float2(1.0f, 0.0f);
            if (lane < half_rot) coef = rope_coefficients(read_only_i32(history_length, b) + s, my_divisor);
            cs[lane] = coef;
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            const float2 t = cs[g * VEC + e];
            c[e] = t.x;
            sn[e] = t.y;
        }
    }
    if (!live) return;

    float x0[VEC], x1[VEC];
    Elem<T>::unpack(lo, x0);
    Elem<T>::unpack(hi, x1);
    if (BIAS) {
        float b0[VEC], b1[VEC];
        Elem<T>::unpack(blo, b0);
        Elem<T>::unpack(bhi, b1);
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            x0[e] += b0[e];
            x1[e] += b1[e];
        }
    }
    T* dst;        // row in the padded q / k / v buffer (k and v may be absent when appending)
    T* cache = nullptr;  // row in the KV cache
    bool rotate = true;
    if (h < head_num) {
        dst = q + (((size_t)b * head_num + h) * seq_len + s) * HS;
    } else {
        const bool is_k = h < head_num + kv_head_num;
        const int kvh = is_k ? h - head_num : h - head_num - kv_head_num;
        T* plane = is_k ? k : v;
        dst = plane ? plane + (((size_t)b * kv_head_num + kvh) * seq_len + s) * HS : nullptr;
        rotate = is_k;
        const long long row = append_row(ap, history_length, b, s);
        if (row >= 0)
            cache = (is_k ? ap.k_cache : ap.v_cache) +
                    (((size_t)b * kv_head_num + kvh) * (size_t)ap.max_seq_len + (size_t)row) * HS;
    }
    float y0[VEC], y1[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) {
        const bool r = rotate && (g * VEC + e) < half_rot;
        float r0, r1;
        rotate_pair(c[e], sn[e], x0[e], x1[e], r0, r1);
        y0[e] = r ? r0 : x0[e];
        y1[e] = r ? r1 : x1[e];
    }
    const vec16 out0 = Elem<T>::pack(y0), out1 = Elem<T>::pack(y1);
    if (dst) {
        store16_sel<ST>(dst + col, out0);
        store16_sel<ST>(dst + HALF + col, out1);
    }
    if (cache) {
        store16_sel<ST>(cache + col, out0);
        store16_sel<ST>(cache + HALF + col, out1);
    }
}

// fp16 heads of 64 elements: a head row is 128 bytes = 8 lanes x 16 bytes, so with one vector per lane
// every load and store instruction of a wave covers 8 whole rows (the general kernel above, whose
// lanes own a half-row vector and its partner 64 bytes further on, moves half rows per instruction
// at this head size: 51-57 % of the peak bandwidth against 57-65 % here).  The rotation partner
// d +- 32 sits 4 lanes away: two DPP row rotations, each enabled for the lane banks it serves, fetch
// it in the VALU.  Same arithmetic per element as rotate_pair(): bit-identical to the other kernels.
// (Measured and not kept: two consecutive tokens per wave in neighbouring lane groups, so that stores
// cover 256 contiguous bytes as with 128-element heads -- 6-10 % slower.)
// grid = (tokens, groups of 8 * WAVES heads).
template <int ST, int WAVES>
__global__ __launch_bounds__(kWave * WAVES) void qkv_rope_rows64_f16(
    __half* __restrict__ q, __half* __restrict__ k, __half* __restrict__ v,
    const __half* __restrict__ qkv, const __half* __restrict__ bias,
    const int32_t* __restrict__ padding_offset, const int32_t* __restrict__ history_length,
    unsigned positions, FastDiv seq, int head_num, int kv_head_num, int half_rot, RopeDivisors tab,
    KvAppend<__half> ap) {
    constexpr int HS = 64, HALF = 32, VEC = 8, LANES_PER_ROW = 8, HEADS_PER_WAVE = kWave / LANES_PER_ROW;
    const int seq_len = (int)seq.d;
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int token = (int)blockIdx.x;
    const int g = lane % LANES_PER_ROW;   // column group: elements 8 g .. 8 g + 7 of the row
    const int slot = lane / LANES_PER_ROW;
    const int qkv_heads = head_num + 2 * kv_head_num;
    const int h = ((int)blockIdx.y * WAVES + wave) * HEADS_PER_WAVE + slot;
    const bool live = h < qkv_heads;
    const int col = g * VEC;
    vec16 raw, braw;
    if (live) {
        raw = load16_stream(qkv + ((size_t)token * (size_t)qkv_heads + h) * HS + col);
        if (bias) braw = load16(bias + (size_t)h * HS + col);
    }
    const long long p = (long long)token + (long long)read_only_i32(padding_offset, (int)token);
    if (p < 0 || p >= (long long)positions) return;  // workgroup-uniform
    unsigned ub, us;
    seq.divmod((unsigned)p, ub, us);
    const int b = (int)ub, s = (int)us;

    // (cos, sin) of the token's pairs: once per workgroup, by its first wave (as in qkv_rope_wave)
    const int block_first = (int)blockIdx.y * WAVES * HEADS_PER_WAVE;
    float c[VEC], sn[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) { c[e] = 1.0f; sn[e] = 0.0f; }
    if (block_first < head_num + kv_head_num) {  // workgroup-uniform
        __shared__ float2 cs[HALF];
        if (wave == 0 && lane < HALF) {
            float2 coef = make_float2(1.0f, 0.0f);
            if (lane < half_rot) coef = rope_coefficients(read_only_i32(history_length, b) + s, tab.div[lane]);
            cs[lane] = coef;
        }
        __syncthreads();
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            const float2 t = cs[(g & 3) * VEC + e];   // pair index d = element index modulo 32
            c[e] = t.x;
            sn[e] = t.y;
        }
    }
    if (!live) return;

    float x[VEC];
    Elem<__half>::unpack(raw, x);
    if (bias) {
        float bv[VEC];
        Elem<__half>::unpack(braw, bv);
#pragma unroll
        for (int e = 0; e < VEC; e++) x[e] += bv[e];
    }
    __half* dst;
    __half* cache = nullptr;
    bool rotate = true;
    if (h < head_num) {
        dst = q + (((size_t)b * head_num + h) * seq_len + s) * HS;
    } else {
        const bool is_k = h < head_num + kv_head_num;
        const int kvh = is_k ? h - head_num : h - head_num - kv_head_num;
        __half* plane = is_k ? k : v;
        dst = plane ? plane + (((size_t)b * kv_head_num + kvh) * seq_len + s) * HS : nullptr;
        rotate = is_k;
        const long long row = append_row(ap, history_length, b, s);
        if (row >= 0)
            cache = (is_k ? ap.k_cache : ap.v_cache) +
                    (((size_t)b * kv_head_num + kvh) * (size_t)ap.max_seq_len + (size_t)row) * HS;
    }
    const bool upper = g >= 4;   // this lane holds x[d + 32]; its partner, 4 lanes down, holds x[d]
    float y[VEC];
#pragma unroll
    for (int e = 0; e < VEC; e++) {
        // partner = the lane 4 further on (lower half rows) or 4 further back (upper half rows).  A row
        // rotation by n hands lane i the value of lane (i - n) mod 16: row_ror:12 serves lane banks 0
        // and 2 of each row of 16 (they read lane i + 4), row_ror:4 banks 1 and 3 (lane i - 4)
        unsigned other = __builtin_amdgcn_update_dpp(0u, __float_as_uint(x[e]), 0x12C, 0xf, 0x5, false);
        other = __builtin_amdgcn_update_dpp(other, __float_as_uint(x[e]), 0x124, 0xf, 0xA, false);
        const float xo = __uint_as_float(other);
        const bool r = rotate && ((g & 3) * VEC + e) < half_rot;
        // lower: c x[d] - s x[d + 32];  upper: c x[d + 32] + s x[d]   (rotate_pair, one half each)
        const float rot = upper ? __fmaf_rn(c[e], x[e], sn[e] * xo) : __fmaf_rn(c[e], x[e], -(sn[e] * xo));
        y[e] = r ? rot : x[e];
    }
    const vec16 out = Elem<__half>::pack(y);
    if (dst) store16_sel<ST>(dst + col, out);
    if (cache) store16_sel<ST>(cache + col, out);
}

// The common LLaMA shape (fp16, head size 128 fully rotated, q and kv head counts multiples of 4)
// with as few instructions per wave as the arithmetic allows, because at one 16-byte vector per
// lane a wave moves only 1 KiB and anything above ~100 vector instructions per wave shows up in
// the run time.  One vector per lane: 512 threads carry a group of 32 heads of one token (all q, all
// k or all v, unless SPLIT), every load and store instruction of a wave covers 4 whole head rows.  The
// rotation partner (d +- 64) is 8 lanes away and comes through a DPP row rotation; (cos, sin) are
// evaluated once per workgroup by its first wave and stored twice, as (c, -s) for the lower and
// (c, s) for the upper half of a row, so that both halves run out = c * x + t * partner; row,
// plane and sequence arithmetic is wave-uniform (scalar).  Same operations per element as
// rotate_pair(), so the results are bit-identical to the other kernels of this file.  BIAS is a
// template argument so that each variant has a fixed sequence of loads and the compiler's waits
// are exact for it; so is APPEND (k and v rows also, or only, into the KV cache).
// SPLIT = false: head counts in multiples of 32, so a workgroup's 32 heads belong to one plane and all
// placement arithmetic is workgroup-uniform.  SPLIT = true: head counts in multiples of 4 (grouped-query
// shapes, 40-head models): each wave places its own 4 heads, the q / k / v boundaries and the end of the
// token's heads may fall between the waves of a workgroup, and a wave without heads reads rows that exist,
// stays until the barrier and leaves.
// `tab` MUST stay the first parameter: first_argument_word() reads it at byte 0 of the argument
// block (the launcher asserts its offset, and a test checks every coefficient through the ABI).
template <int ST, bool BIAS, bool APPEND, bool SPLIT>
__global__ __launch_bounds__(512) void qkv_rope_lean_f16(
    RopeDivisors tab, __half* q, __half* k, __half* v, const __half* qkv, const __half* bias,
    const int32_t* __restrict__ padding_offset, const int32_t* __restrict__ history_length,
    unsigned positions, FastDiv seq, unsigned head_num, unsigned kv_head_num,
    KvAppend<__half> ap) {
    constexpr unsigned ROW_BYTES = 256, GROUP = 32, WAVE_HEADS = 4;
    const unsigned tid = threadIdx.x;
    const unsigned token = blockIdx.x;
    // first head of this workgroup's group: 32 heads, or with SPLIT as many as the launch gave it waves for
    const unsigned group_first = blockIdx.y * (SPLIT ? blockDim.x / (64u / WAVE_HEADS) : GROUP);
    const unsigned qkv_heads = head_num + 2 * kv_head_num;
    // the heads this wave (SPLIT) or this workgroup places start at `first`; `slot` = the lane's 16-byte
    // slot counted from there
    const unsigned first =
        SPLIT ? group_first + (unsigned)__builtin_amdgcn_readfirstlane(tid >> 6) * WAVE_HEADS : group_first;
    const unsigned slot = SPLIT ? (tid & 63u) : tid;
    const bool live = !SPLIT || first < qkv_heads;  // wave-uniform
    const unsigned first_read = live ? first : 0u;

    // loads in the order divisor, streamed row, bias, and kept in it (see first_argument_word)
    const float my_divisor = first_argument_word(tid & 63u);
    (void)tab;
    asm volatile("" ::: "memory");
    const char* src = reinterpret_cast<const char*>(qkv) + ((size_t)token * qkv_heads + first_read) * ROW_BYTES;
    const vec16 raw = load16_stream(src + slot * 16u);
    asm volatile("" ::: "memory");
    vec16 braw;
    if (BIAS) braw = load16(reinterpret_cast<const char*>(bias) + (size_t)first_read * ROW_BYTES + slot * 16u);
    asm volatile("" ::: "memory");  // keeps the loads in front of the lookups below

    const long long p = (long long)token + (long long)read_only_i32(padding_offset, (int)token);
    if (p < 0 || p >= (long long)positions) return;  // workgroup-uniform
    unsigned b, s;
    seq.divmod((unsigned)p, b, s);

    __half* plane;
    unsigned plane_heads, h0;
    const bool rotates = first < head_num + kv_head_num;
    if (first < head_num) {
        plane = q, plane_heads = head_num, h0 = first;
    } else if (rotates) {
        plane = k, plane_heads = kv_head_num, h0 = first - head_num;
    } else {
        plane = v, plane_heads = kv_head_num, h0 = first - head_num - kv_head_num;
    }
    char* dst = reinterpret_cast<char*>(plane) + (((size_t)b * plane_heads + h0) * seq.d + s) * ROW_BYTES;
    const unsigned lane_offset = (slot >> 4) * (seq.d * ROW_BYTES) + (slot & 15u) * 16u;  // head row, column
    // the same rows in the KV cache (k and v heads only); all of it wave-uniform
    char* cdst = nullptr;
    unsigned cache_lane_offset = 0;
    bool idle = !live;  // nothing (more) to write for these heads
    if (APPEND && first >= head_num) {
        const long long row = append_row(ap, history_length, (int)b, (int)s);
        if (row >= 0) {
            cdst = reinterpret_cast<char*>(rotates ? ap.k_cache : ap.v_cache) +
                   (((size_t)b * plane_heads + h0) * (size_t)ap.max_seq_len + (size_t)row) * ROW_BYTES;
            cache_lane_offset = (slot >> 4) * ((unsigned)ap.max_seq_len * ROW_BYTES) + (slot & 15u) * 16u;
        }
        if (plane == nullptr && cdst == nullptr) idle = true;
    }
    if (!idle && !rotates && !BIAS) {  // v heads without bias: a plain move
        if (!APPEND || plane != nullptr) store16_sel<ST>(dst + lane_offset, raw);
        if (APPEND && cdst != nullptr) store16_sel<ST>(cdst + cache_lane_offset, raw);
        idle = true;
    }
    if (!SPLIT && idle) return;  // workgroup-uniform without SPLIT; with it every wave goes on to the barrier
    // the coefficient table first: the first wave evaluates it while every wave's loads are in flight
    // Table layout [j][class][2]: class = tid & 15 names a lane's column and half row (16 classes),
    // j = 0..3 its four 16-byte reads of two (c, t) pairs each; the 16 classes of one j are
    // contiguous (256 bytes = all 64 banks), so the reads of a wave are conflict-free.
    __shared__ float2 cs[4][16][2];
    if (SPLIT ? group_first < head_num + kv_head_num : rotates) {  // workgroup-uniform: its first wave rotates
        if (tid < 64) {
            const float2 coef = rope_coefficients(read_only_i32(history_length, (int)b) + (int)s, my_divisor);
            const unsigned g = tid >> 3, e = tid & 7u;  // pair tid = element e of column group g
            cs[e >> 1][g][e & 1u] = make_float2(coef.x, -coef.y);  // lower half row: c x - s partner
            cs[e >> 1][g + 8][e & 1u] = coef;                      // upper half row: c x + s partner
        }
        __syncthreads();
    }
    if (SPLIT && idle) return;
    float x[8], y[8];
    Elem<__half>::unpack(raw, x);
    if (BIAS) {
        float bv[8];
        Elem<__half>::unpack(braw, bv);
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] += bv[e];
    }
    if (rotates) {
        const unsigned cls = tid & 15u;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float2 t = cs[e >> 1][cls][e & 1];
            const float other = dpp_mov<0x128>(x[e]);  // row_ror:8: the lane 8 further on / back
            y[e] = __fmaf_rn(t.x, x[e], t.y * other);
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) y[e] = x[e];
    }
    const vec16 packed = Elem<__half>::pack(y);
    if (!APPEND || plane != nullptr) store16_sel<ST>(dst + lane_offset, packed);
    if (APPEND && cdst != nullptr) store16_sel<ST>(cdst + cache_lane_offset, packed);
}

// The same design for fp32 rows (head size 128 fully rotated, q and kv head counts multiples of 16, or of 2
// with SPLIT): a head row is 512 bytes = 32 lanes of one 16-byte vector, a wave carries two rows and 512
// threads the 16 heads of one group.  The rotation partner (d +- 64) is 16 lanes away, in the neighbouring row of 16 lanes:
// v_permlane16_swap exchanges the odd rows of one register with the even rows of another, so applied to
// two copies of x it leaves every lane with the value of its even-row neighbour in one result and of its
// odd-row neighbour in the other, and a lane picks the one that is not its own.  Same operations per
// element as rotate_pair(): bit-identical to qkv_rope_wave<float, ...>, which this replaces for that shape
// (two vectors per lane there).
// `tab` MUST stay the first parameter (first_argument_word).
template <int ST, bool BIAS, bool APPEND, bool SPLIT>
__global__ __launch_bounds__(512) void qkv_rope_lean_f32(
    RopeDivisors tab, float* q, float* k, float* v, const float* qkv, const float* bias,
    const int32_t* __restrict__ padding_offset, const int32_t* __restrict__ history_length,
    unsigned positions, FastDiv seq, unsigned head_num, unsigned kv_head_num, KvAppend<float> ap) {
    constexpr unsigned ROW_BYTES = 512, GROUP = 16, WAVE_HEADS = 2;
    const unsigned tid = threadIdx.x;
    const unsigned token = blockIdx.x;
    const unsigned group_first = blockIdx.y * (SPLIT ? blockDim.x / (64u / WAVE_HEADS) : GROUP);
    const unsigned qkv_heads = head_num + 2 * kv_head_num;
    // SPLIT (head counts in multiples of 2 instead of 16): every wave places its own two heads
    const unsigned first =
        SPLIT ? group_first + (unsigned)__builtin_amdgcn_readfirstlane(tid >> 6) * WAVE_HEADS : group_first;
    const unsigned slot = SPLIT ? (tid & 63u) : tid;
    const bool live = !SPLIT || first < qkv_heads;  // wave-uniform
    const unsigned first_read = live ? first : 0u;

    const float my_divisor = first_argument_word(tid & 63u);
    (void)tab;
    asm volatile("" ::: "memory");
    const char* src = reinterpret_cast<const char*>(qkv) + ((size_t)token * qkv_heads + first_read) * ROW_BYTES;
    const vec16 raw = load16_stream(src + slot * 16u);
    asm volatile("" ::: "memory");
    vec16 braw;
    if (BIAS) braw = load16(reinterpret_cast<const char*>(bias) + (size_t)first_read * ROW_BYTES + slot * 16u);
    asm volatile("" ::: "memory");

    const long long p = (long long)token + (long long)read_only_i32(padding_offset, (int)token);
    if (p < 0 || p >= (long long)positions) return;  // workgroup-uniform
    unsigned b, s;
    seq.divmod((unsigned)p, b, s);

    float* plane;
    unsigned plane_heads, h0;
    const bool rotates = first < head_num + kv_head_num;
    if (first < head_num) {
        plane = q, plane_heads = head_num, h0 = first;
    } else if (rotates) {
        plane = k, plane_heads = kv_head_num, h0 = first - head_num;
    } else {
        plane = v, plane_heads = kv_head_num, h0 = first - head_num - kv_head_num;
    }
    char* dst = reinterpret_cast<char*>(plane) + (((size_t)b * plane_heads + h0) * seq.d + s) * ROW_BYTES;
    const unsigned lane_offset = (slot >> 5) * (seq.d * ROW_BYTES) + (slot & 31u) * 16u;  // head row, column
    char* cdst = nullptr;
    unsigned cache_lane_offset = 0;
    bool idle = !live;  // nothing (more) to write for these heads
    if (APPEND && first >= head_num) {
        const long long row = append_row(ap, history_length, (int)b, (int)s);
        if (row >= 0) {
            cdst = reinterpret_cast<char*>(rotates ? ap.k_cache : ap.v_cache) +
                   (((size_t)b * plane_heads + h0) * (size_t)ap.max_seq_len + (size_t)row) * ROW_BYTES;
            cache_lane_offset = (slot >> 5) * ((unsigned)ap.max_seq_len * ROW_BYTES) + (slot & 31u) * 16u;
        }
        if (plane == nullptr && cdst == nullptr) idle = true;
    }
    if (!idle && !rotates && !BIAS) {  // v heads without bias: a plain move
        if (!APPEND || plane != nullptr) store16_sel<ST>(dst + lane_offset, raw);
        if (APPEND && cdst != nullptr) store16_sel<ST>(cdst + cache_lane_offset, raw);
        idle = true;
    }
    if (!SPLIT && idle) return;  // workgroup-uniform without SPLIT; with it every wave goes on to the barrier
    // Table layout [j][class][2]: class = tid & 31 names a lane's column and half row (16 classes of the
    // lower half row with (c, -s), 16 of the upper with (c, s)), j = 0..1 its two 16-byte reads of two
    // (c, t) pairs each; the 32 classes of one j are contiguous
    __shared__ float2 cs[2][32][2];
    if (SPLIT ? group_first < head_num + kv_head_num : rotates) {  // workgroup-uniform: its first wave rotates
        if (tid < 64) {
            const float2 coef = rope_coefficients(read_only_i32(history_length, (int)b) + (int)s, my_divisor);
            const unsigned g = tid >> 2, e = tid & 3u;  // pair tid = element e of column group g
            cs[e >> 1][g][e & 1u] = make_float2(coef.x, -coef.y);
            cs[e >> 1][g + 16][e & 1u] = coef;
        }
        __syncthreads();
    }
    if (SPLIT && idle) return;
    float x[4], y[4];
    Elem<float>::unpack(raw, x);
    if (BIAS) {
        float bv[4];
        Elem<float>::unpack(braw, bv);
#pragma unroll
        for (int e = 0; e < 4; e++) x[e] += bv[e];
    }
    if (rotates) {
        const unsigned cls = tid & 31u;
        const bool upper = (tid & 16u) != 0;  // odd row of 16 lanes: holds x[d + 64], its partner sits one row down
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float2 t = cs[e >> 1][cls][e & 1];
            const unsigned bits = __float_as_uint(x[e]);
            const auto r = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
            // r[0]: every row pair holds its even row's values, r[1]: its odd row's
            const float other = __uint_as_float(upper ? r[0] : r[1]);
            y[e] = __fmaf_rn(t.x, x[e], t.y * other);
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) y[e] = x[e];
    }
    const vec16 packed = Elem<float>::pack(y);
    if (!APPEND || plane != nullptr) store16_sel<ST>(dst + lane_offset, packed);
    if (APPEND && cdst != nullptr) store16_sel<ST>(cdst + cache_lane_offset, packed);
}

// The same design for 64-element heads (fp16, fully rotated, q and kv head counts multiples of 8).  A head
// row is 128 bytes = 8 lanes; a wave carries 8 consecutive heads of one plane (q, k or v: wave-uniform), four
// waves one token's group of 32 heads, and a workgroup of 512 threads TWO tokens, so that its first wave's
// 64 lanes evaluate the 2 x 32 (cos, sin) pairs in one go -- per byte the same coefficient work as the
// 128-element kernel.  Inside each row of 16 lanes the layout is [row A low | row B low | row A high |
// row B high] (4 lanes = 64 bytes each), which puts a lane's rotation partner exactly 8 lanes away: one DPP
// row rotation, as above, instead of two with complementary bank masks.  Every load and store instruction
// of a wave still covers 1 KiB of whole rows.  Waves without work (odd token count, padded position, head
// group beyond the last head) stay until the barrier and then leave.
// `tab` MUST stay the first parameter (first_argument_word).
template <int ST, bool BIAS, bool APPEND>
__global__ __launch_bounds__(512) void qkv_rope_lean64_f16(
    RopeDivisors tab, __half* q, __half* k, __half* v, const __half* qkv, const __half* bias,
    const int32_t* __restrict__ padding_offset, const int32_t* __restrict__ history_length,
    unsigned positions, FastDiv seq, unsigned token_num, unsigned head_num, unsigned kv_head_num,
    KvAppend<__half> ap) {
    constexpr unsigned ROW_BYTES = 128;
    const unsigned tid = threadIdx.x;
    const unsigned which = __builtin_amdgcn_readfirstlane(tid >> 8);        // first or second token
    const unsigned w = __builtin_amdgcn_readfirstlane((tid >> 6) & 3u);     // wave inside the token
    const unsigned token = blockIdx.x * 2u + which;
    const unsigned qkv_heads = head_num + 2 * kv_head_num;
    const unsigned hw = blockIdx.y * 32u + w * 8u;                          // first head of this wave
    bool live = token < token_num && hw < qkv_heads;                        // wave-uniform
    const unsigned l = tid & 15u;
    const unsigned head_in_wave = ((tid & 63u) >> 4) * 2u + ((l >> 2) & 1u);
    const unsigned g = ((l >> 3) << 2) | (l & 3u);                          // 16-byte column of the row
    const unsigned in_block = head_in_wave * ROW_BYTES + g * 16u;

    const float my_divisor = first_argument_word(tid & 31u);
    (void)tab;
    asm volatile("" ::: "memory");
    // unconditional loads (a wave without work reads rows that exist and discards them): with a load
    // inside a branch the compiler can no longer count the outstanding ones and waits for all of them
    // where the first wave only needs its divisor
    const unsigned token_c = token < token_num ? token : blockIdx.x * 2u;
    const unsigned hw_c = hw < qkv_heads ? hw : 0u;
    const vec16 raw =
        load16_stream(reinterpret_cast<const char*>(qkv) + ((size_t)token_c * qkv_heads + hw_c) * ROW_BYTES + in_block);
    asm volatile("" ::: "memory");
    vec16 braw;
    if (BIAS) braw = load16(reinterpret_cast<const char*>(bias) + (size_t)hw_c * ROW_BYTES + in_block);
    asm volatile("" ::: "memory");

    // Both tokens' positions and timesteps through scalar loads, in every wave: they run beside the vector
    // loads above (vector memory returns in issue order, so a vector load of the padding offset would only
    // come back behind the rows, and the first wave's evaluation with it).
    const unsigned tok_a = blockIdx.x * 2u, tok_b = tok_a + 1u;
    const long long p_a = (long long)tok_a + (long long)read_only_i32(padding_offset, (int)tok_a);
    const long long p_b = tok_b < token_num ? (long long)tok_b + (long long)read_only_i32(padding_offset, (int)tok_b) : -1;
    const bool ok_a = p_a >= 0 && p_a < (long long)positions, ok_b = p_b >= 0 && p_b < (long long)positions;
    unsigned b_a = 0, s_a = 0, b_b = 0, s_b = 0;
    if (ok_a) seq.divmod((unsigned)p_a, b_a, s_a);
    if (ok_b) seq.divmod((unsigned)p_b, b_b, s_b);
    live = live && (which ? ok_b : ok_a);
    const unsigned b = which ? b_b : b_a, s = which ? s_b : s_a;

    // Table layout [token][j][class][2]: class = the lane's column g (8 classes: 4 of the lower half row
    // with (c, -s), 4 of the upper with (c, s)), j = 0..3 its four 16-byte reads of two (c, t) pairs each
    __shared__ float2 cs[2][4][8][2];
    if (blockIdx.y * 32u < head_num + kv_head_num) {  // workgroup-uniform: some wave here rotates
        if (tid < 64) {
            // b_a / b_b are 0 for a token without a position: both loads unconditional, so they overlap
            const int h_a = read_only_i32(history_length, (int)b_a), h_b = read_only_i32(history_length, (int)b_b);
            const int t_a = h_a + (int)s_a, t_b = h_b + (int)s_b;
            const float2 coef = rope_coefficients((tid & 32u) ? t_b : t_a, my_divisor);
            const unsigned d = tid & 31u, gg = d >> 3, e = d & 7u;  // pair d = element e of column group gg
            cs[tid >> 5][e >> 1][gg][e & 1u] = make_float2(coef.x, -coef.y);
            cs[tid >> 5][e >> 1][gg + 4][e & 1u] = coef;
        }
        __syncthreads();
    }
    if (!live) return;

    __half* plane;
    unsigned plane_heads, h0;
    const bool rotates = hw < head_num + kv_head_num;
    if (hw < head_num) {
        plane = q, plane_heads = head_num, h0 = hw;
    } else if (rotates) {
        plane = k, plane_heads = kv_head_num, h0 = hw - head_num;
    } else {
        plane = v, plane_heads = kv_head_num, h0 = hw - head_num - kv_head_num;
    }
    char* dst = reinterpret_cast<char*>(plane) + (((size_t)b * plane_heads + h0) * seq.d + s) * ROW_BYTES;
    const unsigned lane_offset = head_in_wave * (seq.d * ROW_BYTES) + g * 16u;
    char* cdst = nullptr;
    unsigned cache_lane_offset = 0;
    if (APPEND && hw >= head_num) {
        const long long row = append_row(ap, history_length, (int)b, (int)s);
        if (row >= 0) {
            cdst = reinterpret_cast<char*>(rotates ? ap.k_cache : ap.v_cache) +
                   (((size_t)b * plane_heads + h0) * (size_t)ap.max_seq_len + (size_t)row) * ROW_BYTES;
            cache_lane_offset = head_in_wave * ((unsigned)ap.max_seq_len * ROW_BYTES) + g * 16u;
        }
        if (plane == nullptr && cdst == nullptr) return;
    }

    if (!rotates && !BIAS) {  // v heads without bias: a plain move
        if (!APPEND || plane != nullptr) store16_sel<ST>(dst + lane_offset, raw);
        if (APPEND && cdst != nullptr) store16_sel<ST>(cdst + cache_lane_offset, raw);
        return;
    }
    float x[8], y[8];
    Elem<__half>::unpack(raw, x);
    if (BIAS) {
        float bv[8];
        Elem<__half>::unpack(braw, bv);
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] += bv[e];
    }
    if (rotates) {
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float2 t = cs[which][e >> 1][g][e & 1];
            const float other = dpp_mov<0x128>(x[e]);  // row_ror:8: the other half of the same head row
            y[e] = __fmaf_rn(t.x, x[e], t.y * other);
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) y[e] = x[e];
    }
    const vec16 packed = Elem<__half>::pack(y);
    if (!APPEND || plane != nullptr) store16_sel<ST>(dst + lane_offset, packed);
    if (APPEND && cdst != nullptr) store16_sel<ST>(cdst + cache_lane_offset, packed);
}

// first_argument_word() reads the divisor table at byte 0 of the kernel's argument block, where the
// ABI puts the first explicit parameter: fail the build if that is ever something else.
template <typename F>
struct FirstParameter;
template <typename A0, typename... A>
struct FirstParameter<void (*)(A0, A...)> {
    using type = A0;
};
static_assert(std::is_same<FirstParameter<decltype(&qkv_rope_lean_f16<kStorePlain, false, false, false>)>::type,
                           RopeDivisors>::value &&
                  offsetof(RopeDivisors, div) == 0,
              "qkv_rope_lean_f16 must take the divisor table as its first parameter");
static_assert(std::is_same<FirstParameter<decltype(&qkv_rope_lean64_f16<kStorePlain, false, false>)>::type,
                           RopeDivisors>::value,
              "qkv_rope_lean64_f16 must take the divisor table as its first parameter");
static_assert(std::is_same<FirstParameter<decltype(&qkv_rope_lean_f32<kStorePlain, false, false, false>)>::type,
                           RopeDivisors>::value,
              "qkv_rope_lean_f32 must take the divisor table as its first parameter");
static_assert(std::is_same<FirstParameter<decltype(&qkv_rope_wave<float, 128, kStorePlain, 4, false>)>::type,
                           RopeDivisors>::value,
              "qkv_rope_wave must take the divisor table as its first parameter");

// Any (even) head size and any alignment: one workgroup per token, one lane per rotation pair.
template <typename T>
__global__ __launch_bounds__(kBlock) void qkv_rope_generic(
    T* q, T* k, T* v, const T* qkv, const T* bias, const int32_t* padding_offset,
    const int32_t* history_length, int batch, int seq_len, int head_num, int kv_head_num,
    int head_size, int half_rot, RopeDivisors tab, KvAppend<T> ap) {
    const int token = blockIdx.x;
    const long long p = (long long)token + (long long)read_only_i32(padding_offset, (int)token);
    if (p < 0 || p >= (long long)batch * (long long)seq_len) return;
    const int b = (int)(p / seq_len);
    const int s = (int)(p % seq_len);
    const int timestep = read_only_i32(history_length, b) + s;
    const long long cache_row = append_row(ap, history_length, b, s);
    const int half = head_size / 2;
    const int qkv_heads = head_num + 2 * kv_head_num;
    const T* row = qkv + (size_t)token * (size_t)qkv_heads * head_size;
    const int pairs = qkv_heads * half;
    for (int i = threadIdx.x; i < pairs; i += kBlock) {
        const int h = i / half;
        const int d = i % half;
        float x0 = Elem<T>::to_f32(row[(size_t)h * head_size + d]);
        float x1 = Elem<T>::to_f32(row[(size_t)h * head_size + half + d]);
        if (bias) {
            x0 += Elem<T>::to_f32(bias[(size_t)h * head_size + d]);
            x1 += Elem<T>::to_f32(bias[(size_t)h * head_size + half + d]);
        }
        T* dst;
        T* cache = nullptr;
        bool rotate = d < half_rot;
        if (h < head_num) {
            dst = q + (((size_t)b * head_num + h) * seq_len + s) * head_size;
        } else {
            const bool is_k = h < head_num + kv_head_num;
            const int kvh = is_k ? h - head_num : h - head_num - kv_head_num;
            T* plane = is_k ? k : v;
            dst = plane ? plane + (((size_t)b * kv_head_num + kvh) * seq_len + s) * head_size : nullptr;
            rotate = rotate && is_k;
            if (cache_row >= 0)
                cache = (is_k ? ap.k_cache : ap.v_cache) +
                        (((size_t)b * kv_head_num + kvh) * (size_t)ap.max_seq_len + (size_t)cache_row) * head_size;
        }
        float y0 = x0, y1 = x1;
        if (rotate) {
            const float2 coef = rope_coefficients(timestep, tab.div[d]);
            rotate_pair(coef.x, coef.y, x0, x1, y0, y1);
        }
        const T o0 = Elem<T>::from_f32(y0), o1 = Elem<T>::from_f32(y1);
        if (dst) {
            dst[d] = o0;
            dst[half + d] = o1;
        }
        if (cache) {
            cache[d] = o0;
            cache[half + d] = o1;
        }
    }
}

// Decode-phase RoPE, in place on packed rows [batch, head_num + 2 kv_head_num, head_size]
// (src/kernels/qkv_bias_and_RoPE.cu:352-390, launcher :404-434): rotate-half on every q and k head
// at timestep step - 1 (:380).  Same lane layout as the prefill kernel: a wave owns kWave / G heads of
// one row, evaluates the 64 (cos, sin) pairs once and shares them through wave-private LDS.
// Each k head is rotated once (the reference rotates k head q / (head_num / kv_head_num) from every q
// block, which only coincides with this when kv_head_num == head_num, the one case it accepts).
//
// The same kernels also run the fused decode step (DecodeExtras): the QKV bias added first, and the
// rotated k row and the v row of sequence b appended to cache[b, head, history_length[b], :] -- what
// launchConcatKVCache does for a one-token query (src/kernels/concat_past_kv.cu:7-73) -- so that a
// decode step needs one launch instead of three launch-bound ones.  With all extras absent only the
// q and k heads are touched, exactly as before.
template <typename T>
struct DecodeExtras {
    const T* bias;                   // [(head_num + 2 kv_head_num) * head_size] or NULL
    T* k_cache;                      // layer slice [batch, kv_head_num, max_seq_len, head_size] or NULL
    T* v_cache;
    const int32_t* history_length;   // [batch]; read only when appending
    int max_seq_len;
};

template <typename T, int HS>
__global__ __launch_bounds__(kBlock) void rope_decode_wave(T* __restrict__ qkv, int head_num,
                                                           int kv_head_num, int timestep,
                                                           int half_rot, RopeDivisors tab,
                                                           DecodeExtras<T> ex) {
    constexpr int VEC = Elem<T>::kVec;
    constexpr int HALF = HS / 2;
    constexpr int G = HALF / VEC;
    constexpr int HEADS_PER_WAVE = kWave / G;
    constexpr int WAVES = kBlock / kWave;
    const int lane = threadIdx.x % kWave;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const int g = lane % G;
    const int slot = lane / G;
    const int rotated_heads = head_num + kv_head_num;
    const bool extras = ex.bias != nullptr || ex.k_cache != nullptr;
    const int covered = extras ? rotated_heads + kv_head_num : rotated_heads;  // v heads only with extras
    const int wave_first = ((int)blockIdx.y * WAVES + wave) * HEADS_PER_WAVE;
    if (wave_first >= covered) return;  // wave-uniform
    const int h = wave_first + slot;
    const bool live = h < covered;
    const int b = (int)blockIdx.x;
    T* p = qkv + ((size_t)b * (size_t)(head_num + 2 * kv_head_num) + (live ? h : 0)) * HS + g * VEC;
    vec16 lo, hi, blo, bhi;
    if (live) {
        lo = load16(p);
        hi = load16(p + HALF);
        if (ex.bias) {
            blo = load16(ex.bias + (size_t)h * HS + g * VEC);
            bhi = load16(ex.bias + (size_t)h * HS + HALF + g * VEC);
        }
    }
    // timestep < 0: each sequence at its own position history_length[b] (a batch of ragged histories)
    const int t = timestep >= 0 ? timestep : read_only_i32(ex.history_length, b);
    __shared__ float2 cs[WAVES][HALF];
    if (lane < HALF) {
        float2 coef = make_float2(1.0f, 0.0f);
        if (lane < half_rot) coef = rope_coefficients(t, tab.div[lane]);
        cs[wave][lane] = coef;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if (!live) return;
    const bool is_v = h >= rotated_heads;
    float x0[VEC], x1[VEC], y0[VEC], y1[VEC];
    Elem<T>::unpack(lo, x0);
    Elem<T>::unpack(hi, x1);
    if (ex.bias) {
        float b0[VEC], b1[VEC];
        Elem<T>::unpack(blo, b0);
        Elem<T>::unpack(bhi, b1);
#pragma unroll
        for (int e = 0; e < VEC; e++) {
            x0[e] += b0[e];
            x1[e] += b1[e];
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; e++) {
        const float2 t = cs[wave][g * VEC + e];
        const bool r = !is_v && (g * VEC + e) < half_rot;
        float r0, r1;
        rotate_pair(t.x, t.y, x0[e], x1[e], r0, r1);
        y0[e] = r ? r0 : x0[e];
        y1[e] = r ? r1 : x1[e];
    }
    const vec16 out0 = Elem<T>::pack(y0), out1 = Elem<T>::pack(y1);
    if (!is_v || ex.bias) {  // a v row without bias is unchanged
        store16(p, out0);
        store16(p + HALF, out1);
    }
    if (ex.k_cache && h >= head_num) {
        const long long row = read_only_i32(ex.history_length, b);
        if (row >= 0 && row < ex.max_seq_len) {
            const int kvh = is_v ? h - rotated_heads : h - head_num;
            T* c = (is_v ? ex.v_cache : ex.k_cache) +
                   (((size_t)b * kv_head_num + kvh) * (size_t)ex.max_seq_len + (size_t)row) * HS + g * VEC;
            store16(c, out0);
            store16(c + HALF, out1);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void rope_decode_generic(T* qkv, int head_num, int kv_head_num,
                                                              int head_size, int timestep,
                                                              int half_rot, RopeDivisors tab,
                                                              DecodeExtras<T> ex) {
    const int half = head_size / 2;
    const int b = (int)blockIdx.x;
    T* row = qkv + (size_t)b * (size_t)(head_num + 2 * kv_head_num) * head_size;
    const int rotated_heads = head_num + kv_head_num;
    const bool extras = ex.bias != nullptr || ex.k_cache != nullptr;
    const int covered = extras ? rotated_heads + kv_head_num : rotated_heads;
    // without extras only the rotated pairs are touched; with them every pair of every covered head
    const int per_head = extras ? half : half_rot;
    const int pairs = covered * per_head;
    const int t = timestep >= 0 ? timestep : read_only_i32(ex.history_length, b);
    long long cache_row = -1;
    if (ex.k_cache) {
        cache_row = read_only_i32(ex.history_length, b);
        if (cache_row < 0 || cache_row >= ex.max_seq_len) cache_row = -1;
    }
    for (int i = threadIdx.x; i < pairs; i += kBlock) {
        const int h = i / per_head, d = i % per_head;
        const bool is_v = h >= rotated_heads;
        T* p = row + (size_t)h * head_size + d;
        float x0 = Elem<T>::to_f32(p[0]), x1 = Elem<T>::to_f32(p[half]);
        if (ex.bias) {
            x0 += Elem<T>::to_f32(ex.bias[(size_t)h * head_size + d]);
            x1 += Elem<T>::to_f32(ex.bias[(size_t)h * head_size + half + d]);
        }
        float y0 = x0, y1 = x1;
        if (!is_v && d < half_rot) {
            const float2 coef = rope_coefficients(t, tab.div[d]);
            rotate_pair(coef.x, coef.y, x0, x1, y0, y1);
        }
        const T o0 = Elem<T>::from_f32(y0), o1 = Elem<T>::from_f32(y1);
        if (!is_v || ex.bias) {
            p[0] = o0;
            p[half] = o1;
        }
        if (cache_row >= 0 && h >= head_num) {
            const int kvh = is_v ? h - rotated_heads : h - head_num;
            T* c = (is_v ? ex.v_cache : ex.k_cache) +
                   (((size_t)b * kv_head_num + kvh) * (size_t)ex.max_seq_len + (size_t)cache_row) * head_size + d;
            c[0] = o0;
            c[half] = o1;
        }
    }
}

// base^(2d/rot) with the C library's powf.  A model calls with one (rot, base) over and over, and
// 128 powf cost about as much host time as the whole launch of a decode step, so each host thread
// keeps the table of its last call.
static void fill_divisors(RopeDivisors& tab, int rot, float base) {
    static thread_local RopeDivisors cached;
    static thread_local int cached_rot = -1;
    static thread_local float cached_base = 0.0f;
    if (cached_rot != rot || cached_base != base) {
        const int half_rot = rot / 2;
        for (int d = 0; d < kMaxHalfRot; d++)
            cached.div[d] = d < half_rot ? powf(base, (float)(2 * d) / (float)rot) : 1.0f;
        cached_rot = rot;
        cached_base = base;
    }
    tab = cached;
}

// bias_ / caches NULL: plain launchRoPE.  Otherwise the fused decode step (see DecodeExtras).
template <typename T>
static int rope_decode(void* qkv_, int batch, int head_num, int kv_head_num, int head_size, int step,
                       int rot, float base, hipStream_t s, const void* bias_ = nullptr,
                       void* k_cache_ = nullptr, void* v_cache_ = nullptr, int layer = 0,
                       int max_seq_len = 0, const int32_t* history_length = nullptr) {
    if (batch < 0 || head_num < 0 || kv_head_num < 0 || head_size < 0 || rot < 0 || layer < 0 || max_seq_len < 0)
        return ISP_ERR_BAD_SHAPE;
    const bool append = k_cache_ != nullptr || v_cache_ != nullptr;
    const bool extras = append || bias_ != nullptr;
    if (batch == 0 || head_size == 0 || head_num + kv_head_num == 0) return ISP_OK;
    if (rot == 0 && !extras) return ISP_OK;
    if (head_size % 2 != 0 || rot % 2 != 0 || rot > head_size) return ISP_ERR_BAD_SHAPE;
    if (rot / 2 > kMaxHalfRot) return ISP_ERR_UNSUPPORTED;
    ISP_REQUIRE_PTR(qkv_);
    T* qkv = static_cast<T*>(qkv_);
    DecodeExtras<T> ex = {static_cast<const T*>(bias_), nullptr, nullptr, history_length, max_seq_len};
    if (append && kv_head_num > 0) {
        ISP_REQUIRE_PTR(k_cache_);
        ISP_REQUIRE_PTR(v_cache_);
        ISP_REQUIRE_PTR(history_length);
        const size_t layer_elems = (size_t)layer * batch * kv_head_num * max_seq_len * head_size;  // concat_past_kv.cu:89
        ex.k_cache = static_cast<T*>(k_cache_) + layer_elems;
        ex.v_cache = static_cast<T*>(v_cache_) + layer_elems;
    }
    RopeDivisors tab;
    fill_divisors(tab, rot, base);
    // step >= 1: every sequence at timestep step - 1 (qkv_bias_and_RoPE.cu:380).  step == 0 (the fused decode step
    // only): each sequence at its own history_length[b], the position its k / v row is appended at -- a batch whose
    // sequences have different histories.  The kernels take that as a negative timestep.
    if (step == 0) ISP_REQUIRE_PTR(history_length);
    if (step < 0) return ISP_ERR_BAD_SHAPE;
    const int timestep = step - 1;
    const int half_rot = rot / 2;
    const int covered = head_num + kv_head_num + ((ex.bias || ex.k_cache) ? kv_head_num : 0);
    dim3 block(kBlock);
    const bool vec_ok = aligned16(qkv) && aligned16(ex.bias) && aligned16(ex.k_cache) && aligned16(ex.v_cache);
    if (vec_ok && (head_size == 128 || head_size == 64) && covered <= 65535) {
        const int hpb = (kWave / ((head_size / 2) / Elem<T>::kVec)) * (kBlock / kWave);
        dim3 grid((unsigned)batch, (unsigned)((covered + hpb - 1) / hpb));
        if (head_size == 128)
            hipLaunchKernelGGL((rope_decode_wave<T, 128>), grid, block, 0, s, qkv, head_num, kv_head_num,
                               timestep, half_rot, tab, ex);
        else
            hipLaunchKernelGGL((rope_decode_wave<T, 64>), grid, block, 0, s, qkv, head_num, kv_head_num,
                               timestep, half_rot, tab, ex);
    } else {
        hipLaunchKernelGGL((rope_decode_generic<T>), dim3((unsigned)batch), block, 0, s, qkv, head_num,
                           kv_head_num, head_size, timestep, half_rot, tab, ex);
    }
    return note_launch(hipGetLastError());
}

// Workgroup shape for the one-vector-per-lane kernels, whose waves carry `wave_heads` whole heads each.
// Head counts in whole groups of eight waves: 8 waves, all of one plane (q, k or v).  Otherwise `split`:
// every wave places its own heads, and the workgroup has the largest number of waves from 8 down to 3 that
// divides the token's waves, so that no wave is launched without heads (36 heads of fp16 in 512-thread
// workgroups, 7 of 16 waves idle, measured 10 % slower than the general kernel).  waves = 0: the head
// counts fit neither, the caller uses the general kernel.
struct LeanShape {
    int waves;
    bool split;
    int groups(int qkv_heads, int wave_heads) const { return (qkv_heads + wave_heads * waves - 1) / (wave_heads * waves); }
};
static LeanShape lean_shape(int head_num, int kv_head_num, int wave_heads) {
    if (head_num % wave_heads != 0 || kv_head_num % wave_heads != 0) return {0, false};
    if (head_num % (8 * wave_heads) == 0 && kv_head_num % (8 * wave_heads) == 0) return {8, false};
    const int token_waves = (head_num + 2 * kv_head_num) / wave_heads;
    for (int w = 8; w >= 3; w--)
        if (token_waves % w == 0) return {w, true};
    return {0, false};
}

// `append`: also (k_ / v_ non-NULL) or only (k_ / v_ NULL) write the k and v rows into the KV cache
// [layers, batch, kv_head_num, max_seq_len, head_size] at layer `layer`.
template <typename T>
static int qkv_rope(void* q_, void* k_, void* v_, const void* qkv_, const void* bias_,
                    const int32_t* padding_offset, const int32_t* history_length,
                    const int32_t* input_length, int batch, int seq_len, int token_num,
                    int head_num, int kv_head_num, int head_size, int rot, float base,
                    hipStream_t s, bool append = false, void* k_cache_ = nullptr,
                    void* v_cache_ = nullptr, int layer = 0, int max_seq_len = 0) {
    // without `append`, input_length is read by the reference kernel but its value is unused
    // (qkv_bias_and_RoPE.cu:161)
    if (append && (layer < 0 || max_seq_len < 0)) return ISP_ERR_BAD_SHAPE;
    if (batch < 0 || seq_len < 0 || token_num < 0 || head_num < 0 || kv_head_num < 0 ||
        head_size < 0 || rot < 0)
        return ISP_ERR_BAD_SHAPE;
    if (token_num == 0 || head_size == 0 || head_num + kv_head_num == 0) return ISP_OK;
    if (batch == 0 || seq_len == 0) return ISP_ERR_BAD_SHAPE;
    if (head_size % 2 != 0 || rot % 2 != 0 || rot > head_size) return ISP_ERR_BAD_SHAPE;
    if (rot / 2 > kMaxHalfRot) return ISP_ERR_UNSUPPORTED;
    if ((long long)head_num + 2ll * kv_head_num > 0x7fffffffll / (head_size > 0 ? head_size : 1))
        return ISP_ERR_UNSUPPORTED;
    ISP_REQUIRE_PTR(qkv_);
    ISP_REQUIRE_PTR(padding_offset);
    ISP_REQUIRE_PTR(history_length);
    if (head_num > 0) ISP_REQUIRE_PTR(q_);
    if (kv_head_num > 0 && !append) {
        ISP_REQUIRE_PTR(k_);
        ISP_REQUIRE_PTR(v_);
    }
    if ((k_ == nullptr) != (v_ == nullptr)) return ISP_ERR_NULL_POINTER;
    T* q = static_cast<T*>(q_);
    T* k = static_cast<T*>(k_);
    T* v = static_cast<T*>(v_);
    const T* qkv = static_cast<const T*>(qkv_);
    const T* bias = static_cast<const T*>(bias_);
    KvAppend<T> ap = {nullptr, nullptr, input_length, max_seq_len};
    if (append && kv_head_num > 0) {
        ISP_REQUIRE_PTR(k_cache_);
        ISP_REQUIRE_PTR(v_cache_);
        ISP_REQUIRE_PTR(input_length);
        // layer offset as in launchConcatKVCache (concat_past_kv.cu:89)
        const size_t layer_elems = (size_t)layer * batch * kv_head_num * max_seq_len * head_size;
        ap.k_cache = static_cast<T*>(k_cache_) + layer_elems;
        ap.v_cache = static_cast<T*>(v_cache_) + layer_elems;
    }

    RopeDivisors tab;
    const int half_rot = rot / 2;
    fill_divisors(tab, rot, base);

    const bool vec_ok = aligned16(q) && aligned16(k) && aligned16(v) && aligned16(qkv) &&
                        (!bias || aligned16(bias)) && aligned16(ap.k_cache) && aligned16(ap.v_cache);
    dim3 grid((unsigned)token_num), block(kBlock);
    hipError_t e;
    const int kind = store_kind(tuning(ISP_TUNE_QKV_STORE), kStoreThrough);
    int waves = tuning(ISP_TUNE_QKV_WAVES);
    if (waves != 1 && waves != 2 && waves != 4) waves = 4;  // 4 measured best (8 and 12 are slower)
#define ISP_QKV_LAUNCH_1(HS, K, W)                                                                 \
    do {                                                                                           \
        constexpr int HPB = (kWave / ((HS / 2) / Elem<T>::kVec)) * W;                              \
        dim3 g2((unsigned)token_num, (unsigned)((head_num + 2 * kv_head_num + HPB - 1) / HPB));    \
        if (bias)                                                                                  \
            hipLaunchKernelGGL((qkv_rope_wave<T, HS, K, W, true>), g2, dim3(kWave * W), 0, s, tab, q,  \
                               k, v, qkv, bias, padding_offset, history_length, positions, fd,     \
                               head_num, kv_head_num, half_rot, ap);                               \
        else                                                                                       \
            hipLaunchKernelGGL((qkv_rope_wave<T, HS, K, W, false>), g2, dim3(kWave * W), 0, s, tab, q, \
                               k, v, qkv, bias, padding_offset, history_length, positions, fd,     \
                               head_num, kv_head_num, half_rot, ap);                               \
    } while (0)
#define ISP_QKV_LAUNCH_K(HS, W)                                                                    \
    do {                                                                                           \
        if (kind == kStoreThrough) ISP_QKV_LAUNCH_1(HS, kStoreThrough, W);                         \
        else if (kind == kStoreStream) ISP_QKV_LAUNCH_1(HS, kStoreStream, W);                      \
        else ISP_QKV_LAUNCH_1(HS, kStorePlain, W);                                                 \
    } while (0)
#define ISP_QKV_LAUNCH_WAVE(HS)                                                                    \
    do {                                                                                           \
        if (waves == 1) ISP_QKV_LAUNCH_K(HS, 1);                                                   \
        else if (waves == 2) ISP_QKV_LAUNCH_K(HS, 2);                                              \
        else ISP_QKV_LAUNCH_K(HS, 4);                                                              \
    } while (0)
    const int head_groups_max = 65535 * 4;  // grid.y limit, 4 heads per workgroup at least
    // the vector kernels keep padded positions in 32 bits and divide by seq_len with a multiply-high
    const bool positions_ok = (unsigned long long)batch * (unsigned long long)seq_len <= 0x7fffffffull;
    const unsigned positions = positions_ok ? (unsigned)batch * (unsigned)seq_len : 0u;
    const FastDiv fd = make_fastdiv((unsigned)seq_len);
    // one-vector-per-lane kernels: 128-element heads fully rotated, head counts that fill whole waves (4 heads
    // in fp16, 2 in fp32), offsets inside a group and positions inside the batch in 32 bits;
    // ISP_TUNE_QKV_WAVES = 1, 2, 4 opts out
    const int waves_knob = tuning(ISP_TUNE_QKV_WAVES);
    const int qkv_heads = head_num + 2 * kv_head_num;
    const int lean_wave_heads = sizeof(T) == 2 ? 4 : 2;
    const LeanShape lean = lean_shape(head_num, kv_head_num, lean_wave_heads);
    const bool lean_ok = vec_ok && head_size == 128 && rot == 128 && lean.waves > 0 &&
                         lean.groups(qkv_heads, lean_wave_heads) <= 65535 &&
                         (unsigned long long)seq_len * 8192ull <= 0xffffffffull &&
                         (unsigned long long)max_seq_len * 8192ull <= 0xffffffffull &&
                         positions_ok && (waves_knob <= 0 || waves_knob >= 8);
    const dim3 lean_grid((unsigned)token_num, (unsigned)(lean_ok ? lean.groups(qkv_heads, lean_wave_heads) : 1));
    const dim3 lean_block(64u * (unsigned)(lean_ok ? lean.waves : 1));
    if (lean_ok && sizeof(T) == 2) {
        __half* qh = reinterpret_cast<__half*>(q);
        __half* kh = reinterpret_cast<__half*>(k);
        __half* vh = reinterpret_cast<__half*>(v);
        const __half* xh = reinterpret_cast<const __half*>(qkv);
        const __half* bh = reinterpret_cast<const __half*>(bias);
        KvAppend<__half> aph = {reinterpret_cast<__half*>(ap.k_cache), reinterpret_cast<__half*>(ap.v_cache),
                                ap.input_length, ap.max_seq_len};
        const bool with_append = aph.k_cache != nullptr;
#define ISP_QKV_LEAN_3(K, B, A, S)                                                                 \
    hipLaunchKernelGGL((qkv_rope_lean_f16<K, B, A, S>), lean_grid, lean_block, 0, s, tab, qh, kh,  \
                       vh, xh, bh, padding_offset, history_length, positions, fd,                  \
                       (unsigned)head_num, (unsigned)kv_head_num, aph)
#define ISP_QKV_LEAN_2(K, B, A)                                                                    \
    do {                                                                                           \
        if (lean.split) ISP_QKV_LEAN_3(K, B, A, true);                                             \
        else ISP_QKV_LEAN_3(K, B, A, false);                                                       \
    } while (0)
#define ISP_QKV_LEAN(K)                                                                            \
    do {                                                                                           \
        if (bh && with_append) ISP_QKV_LEAN_2(K, true, true);                                      \
        else if (bh) ISP_QKV_LEAN_2(K, true, false);                                               \
        else if (with_append) ISP_QKV_LEAN_2(K, false, true);                                      \
        else ISP_QKV_LEAN_2(K, false, false);                                                      \
    } while (0)
        if (kind == kStoreThrough) ISP_QKV_LEAN(kStoreThrough);
        else if (kind == kStoreStream) ISP_QKV_LEAN(kStoreStream);
        else ISP_QKV_LEAN(kStorePlain);
#undef ISP_QKV_LEAN_3
#undef ISP_QKV_LEAN_2
#undef ISP_QKV_LEAN
        e = hipGetLastError();
    } else if (lean_ok) {
        // fp32 rows of 512 bytes: 16 heads per workgroup of 512 threads
        float* qf = reinterpret_cast<float*>(q);
        float* kf = reinterpret_cast<float*>(k);
        float* vf = reinterpret_cast<float*>(v);
        const float* xf = reinterpret_cast<const float*>(qkv);
        const float* bf = reinterpret_cast<const float*>(bias);
        KvAppend<float> apf = {reinterpret_cast<float*>(ap.k_cache), reinterpret_cast<float*>(ap.v_cache),
                               ap.input_length, ap.max_seq_len};
        const bool with_append = apf.k_cache != nullptr;
#define ISP_QKV_LEAN32_3(K, B, A, S)                                                               \
    hipLaunchKernelGGL((qkv_rope_lean_f32<K, B, A, S>), lean_grid, lean_block, 0, s, tab, qf, kf,  \
                       vf, xf, bf, padding_offset, history_length, positions, fd,                  \
                       (unsigned)head_num, (unsigned)kv_head_num, apf)
#define ISP_QKV_LEAN32_2(K, B, A)                                                                  \
    do {                                                                                           \
        if (lean.split) ISP_QKV_LEAN32_3(K, B, A, true);                                           \
        else ISP_QKV_LEAN32_3(K, B, A, false);                                                     \
    } while (0)
#define ISP_QKV_LEAN32(K)                                                                          \
    do {                                                                                           \
        if (bf && with_append) ISP_QKV_LEAN32_2(K, true, true);                                    \
        else if (bf) ISP_QKV_LEAN32_2(K, true, false);                                             \
        else if (with_append) ISP_QKV_LEAN32_2(K, false, true);                                    \
        else ISP_QKV_LEAN32_2(K, false, false);                                                    \
    } while (0)
        if (kind == kStoreThrough) ISP_QKV_LEAN32(kStoreThrough);
        else if (kind == kStoreStream) ISP_QKV_LEAN32(kStoreStream);
        else ISP_QKV_LEAN32(kStorePlain);
#undef ISP_QKV_LEAN32_3
#undef ISP_QKV_LEAN32_2
#undef ISP_QKV_LEAN32
        e = hipGetLastError();
    } else if (vec_ok && positions_ok && head_size == 128 && head_num + 2 * kv_head_num <= head_groups_max) {
        ISP_QKV_LAUNCH_WAVE(128);
        e = hipGetLastError();
    } else if (sizeof(T) == 2 && vec_ok && positions_ok && head_size == 64 && rot == 64 && waves_knob <= 0 &&
               head_num % 8 == 0 && kv_head_num % 8 == 0 && (head_num + 2 * kv_head_num + 31) / 32 <= 65535 &&
               (unsigned long long)seq_len * 128ull * 8ull <= 0xffffffffull &&
               (unsigned long long)max_seq_len * 128ull * 8ull <= 0xffffffffull) {
        // fp16 rows of 128 bytes in whole groups of 8 heads: two tokens per 512-thread workgroup
        const dim3 g2((unsigned)((token_num + 1) / 2), (unsigned)((head_num + 2 * kv_head_num + 31) / 32));
        __half* qh = reinterpret_cast<__half*>(q);
        __half* kh = reinterpret_cast<__half*>(k);
        __half* vh = reinterpret_cast<__half*>(v);
        const __half* xh = reinterpret_cast<const __half*>(qkv);
        const __half* bh = reinterpret_cast<const __half*>(bias);
        KvAppend<__half> aph = {reinterpret_cast<__half*>(ap.k_cache), reinterpret_cast<__half*>(ap.v_cache),
                                ap.input_length, ap.max_seq_len};
        const bool with_append = aph.k_cache != nullptr;
#define ISP_QKV_LEAN64_2(K, B, A)                                                                  \
    hipLaunchKernelGGL((qkv_rope_lean64_f16<K, B, A>), g2, dim3(512), 0, s, tab, qh, kh, vh, xh, bh, \
                       padding_offset, history_length, positions, fd, (unsigned)token_num,         \
                       (unsigned)head_num, (unsigned)kv_head_num, aph)
#define ISP_QKV_LEAN64(K)                                                                          \
    do {                                                                                           \
        if (bh && with_append) ISP_QKV_LEAN64_2(K, true, true);                                    \
        else if (bh) ISP_QKV_LEAN64_2(K, true, false);                                             \
        else if (with_append) ISP_QKV_LEAN64_2(K, false, true);                                    \
        else ISP_QKV_LEAN64_2(K, false, false);                                                    \
    } while (0)
        if (kind == kStoreThrough) ISP_QKV_LEAN64(kStoreThrough);
        else if (kind == kStoreStream) ISP_QKV_LEAN64(kStoreStream);
        else ISP_QKV_LEAN64(kStorePlain);
#undef ISP_QKV_LEAN64_2
#undef ISP_QKV_LEAN64
        e = hipGetLastError();
    } else if (sizeof(T) == 2 && vec_ok && positions_ok && head_size == 64 && (waves_knob <= 0 || waves_knob >= 8) &&
               head_num + 2 * kv_head_num <= head_groups_max) {
        // fp16 rows of 128 bytes: one vector per lane, 8 lanes per row, 4 waves = 32 heads per workgroup
        constexpr int W = 4;
        const dim3 g2((unsigned)token_num, (unsigned)((head_num + 2 * kv_head_num + 8 * W - 1) / (8 * W)));
        KvAppend<__half> aph = {reinterpret_cast<__half*>(ap.k_cache), reinterpret_cast<__half*>(ap.v_cache),
                                ap.input_length, ap.max_seq_len};
#define ISP_QKV_ROWS64(K)                                                                          \
    hipLaunchKernelGGL((qkv_rope_rows64_f16<K, W>), g2, dim3(kWave * W), 0, s,                      \
                       reinterpret_cast<__half*>(q), reinterpret_cast<__half*>(k),                 \
                       reinterpret_cast<__half*>(v), reinterpret_cast<const __half*>(qkv),         \
                       reinterpret_cast<const __half*>(bias), padding_offset, history_length,      \
                       positions, fd, head_num, kv_head_num, half_rot, tab, aph)
        if (kind == kStoreThrough) ISP_QKV_ROWS64(kStoreThrough);
        else if (kind == kStoreStream) ISP_QKV_ROWS64(kStoreStream);
        else ISP_QKV_ROWS64(kStorePlain);
#undef ISP_QKV_ROWS64
        e = hipGetLastError();
    } else if (vec_ok && positions_ok && head_size == 64 && head_num + 2 * kv_head_num <= head_groups_max) {
        ISP_QKV_LAUNCH_WAVE(64);
        e = hipGetLastError();
    } else {
        hipLaunchKernelGGL((qkv_rope_generic<T>), grid, block, 0, s, q, k, v, qkv, bias,
                           padding_offset, history_length, batch, seq_len, head_num, kv_head_num,
                           head_size, half_rot, tab, ap);
        e = hipGetLastError();
    }
    return note_launch(e);
}

}  // namespace isp

extern "C" {

int isp_qkv_bias_rope_transpose_f32(void* q, void* k, void* v, const void* qkv, const void* bias,
                                    const int32_t* padding_offset, const int32_t* history_length,
                                    const int32_t* input_length, int batch, int seq_len,
                                    int token_num, int head_num, int kv_head_num, int head_size,
                                    int rotary_embedding_dim, float rotary_embedding_base,
                                    int max_position_embeddings, int use_dynamic_ntk,
                                    isp_stream_t stream) {
    (void)max_position_embeddings;
    (void)use_dynamic_ntk;
    return isp::qkv_rope<float>(q, k, v, qkv, bias, padding_offset, history_length, input_length,
                                batch, seq_len, token_num, head_num, kv_head_num, head_size,
                                rotary_embedding_dim, rotary_embedding_base,
                                static_cast<hipStream_t>(stream));
}

int isp_qkv_bias_rope_transpose_f16(void* q, void* k, void* v, const void* qkv, const void* bias,
                                    const int32_t* padding_offset, const int32_t* history_length,
                                    const int32_t* input_length, int batch, int seq_len,
                                    int token_num, int head_num, int kv_head_num, int head_size,
                                    int rotary_embedding_dim, float rotary_embedding_base,
                                    int max_position_embeddings, int use_dynamic_ntk,
                                    isp_stream_t stream) {
    (void)max_position_embeddings;
    (void)use_dynamic_ntk;
    return isp::qkv_rope<__half>(q, k, v, qkv, bias, padding_offset, history_length, input_length,
                                 batch, seq_len, token_num, head_num, kv_head_num, head_size,
                                 rotary_embedding_dim, rotary_embedding_base,
                                 static_cast<hipStream_t>(stream));
}

int isp_qkv_bias_rope_transpose_append_f32(void* q, void* k, void* v, void* k_cache, void* v_cache,
                                           int layer, int max_seq_len, const void* qkv,
                                           const void* bias, const int32_t* padding_offset,
                                           const int32_t* history_length,
                                           const int32_t* input_length, int batch, int seq_len,
                                           int token_num, int head_num, int kv_head_num,
                                           int head_size, int rotary_embedding_dim,
                                           float rotary_embedding_base, isp_stream_t stream) {
    return isp::qkv_rope<float>(q, k, v, qkv, bias, padding_offset, history_length, input_length,
                                batch, seq_len, token_num, head_num, kv_head_num, head_size,
                                rotary_embedding_dim, rotary_embedding_base,
                                static_cast<hipStream_t>(stream), true, k_cache, v_cache, layer,
                                max_seq_len);
}

int isp_qkv_bias_rope_transpose_append_f16(void* q, void* k, void* v, void* k_cache, void* v_cache,
                                           int layer, int max_seq_len, const void* qkv,
                                           const void* bias, const int32_t* padding_offset,
                                           const int32_t* history_length,
                                           const int32_t* input_length, int batch, int seq_len,
                                           int token_num, int head_num, int kv_head_num,
                                           int head_size, int rotary_embedding_dim,
                                           float rotary_embedding_base, isp_stream_t stream) {
    return isp::qkv_rope<__half>(q, k, v, qkv, bias, padding_offset, history_length, input_length,
                                 batch, seq_len, token_num, head_num, kv_head_num, head_size,
                                 rotary_embedding_dim, rotary_embedding_base,
                                 static_cast<hipStream_t>(stream), true, k_cache, v_cache, layer,
                                 max_seq_len);
}

int isp_rope_decode_append_f32(void* qkv, const void* bias, void* k_cache, void* v_cache, int layer,
                               int max_seq_len, const int32_t* history_length, int batch,
                               int head_num, int kv_head_num, int head_size, int step,
                               int rotary_embedding_dim, float rotary_embedding_base,
                               isp_stream_t stream) {
    return isp::rope_decode<float>(qkv, batch, head_num, kv_head_num, head_size, step,
                                   rotary_embedding_dim, rotary_embedding_base,
                                   static_cast<hipStream_t>(stream), bias, k_cache, v_cache, layer,
                                   max_seq_len, history_length);
}

int isp_rope_decode_append_f16(void* qkv, const void* bias, void* k_cache, void* v_cache, int layer,
                               int max_seq_len, const int32_t* history_length, int batch,
                               int head_num, int kv_head_num, int head_size, int step,
                               int rotary_embedding_dim, float rotary_embedding_base,
                               isp_stream_t stream) {
    return isp::rope_decode<__half>(qkv, batch, head_num, kv_head_num, head_size, step,
                                    rotary_embedding_dim, rotary_embedding_base,
                                    static_cast<hipStream_t>(stream), bias, k_cache, v_cache, layer,
                                    max_seq_len, history_length);
}

int isp_rope_decode_f32(void* qkv, int batch, int head_num, int kv_head_num, int head_size, int step,
                        int rotary_embedding_dim, float rotary_embedding_base, isp_stream_t stream) {
    return isp::rope_decode<float>(qkv, batch, head_num, kv_head_num, head_size, step,
                                   rotary_embedding_dim, rotary_embedding_base,
                                   static_cast<hipStream_t>(stream));
}

int isp_rope_decode_f16(void* qkv, int batch, int head_num, int kv_head_num, int head_size, int step,
                        int rotary_embedding_dim, float rotary_embedding_base, isp_stream_t stream) {
    return isp::rope_decode<__half>(qkv, batch, head_num, kv_head_num, head_size, step,
                                    rotary_embedding_dim, rotary_embedding_base,
                                    static_cast<hipStream_t>(stream));
}

}  // extern "C"
