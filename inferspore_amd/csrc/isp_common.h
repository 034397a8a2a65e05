// Shared host/device helpers for the gfx950 kernels.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <stdint.h>

#include "inferspore_amd.h"

namespace isp {

constexpr int kWave = 64;     // CDNA wavefront width
constexpr int kBlock = 256;   // threads per workgroup used by every kernel here (4 waves)

// ----------------------------------------------------------------------------- host side

// Records a failed launch for isp_last_hip_error(); returns the status to hand back.
int note_launch(hipError_t e);

// Current value of a tuning knob (isp_tuning_set); 0 means "automatic" for every knob.
int tuning(int knob);

// Wavefronts the current device holds at once (compute units x 32), cached per device.
int resident_waves();

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Widest unit (4, 2 or 1 bytes) that divides `bytes` and the addresses of all the given pointers:
// the copy width of the fallback kernels for rows that are not whole aligned 16-byte vectors.
template <typename... P>
inline int copy_unit(size_t bytes, const P*... ptrs) {
    uintptr_t bits = (uintptr_t)bytes;
    ((bits |= reinterpret_cast<uintptr_t>(ptrs)), ...);
    return (bits & 3u) == 0 ? 4 : (bits & 1u) == 0 ? 2 : 1;
}

#define ISP_REQUIRE_PTR(p)                   \
    do {                                     \
        if ((p) == nullptr) return ISP_ERR_NULL_POINTER; \
    } while (0)

// ----------------------------------------------------------------------------- device side

// 16-byte vector used for every global access on the fast paths (global_load_dwordx4).
struct __attribute__((aligned(16))) vec16 {
    uint32_t w[4];
};

__device__ __forceinline__ vec16 load16(const void* p) {
    return *reinterpret_cast<const vec16*>(p);
}
__device__ __forceinline__ void store16(void* p, const vec16& v) {
    *reinterpret_cast<vec16*>(p) = v;
}
// Streaming variants: data touched once is marked non-temporal so it does not displace the small
// operands (gamma, bias, tables) that every row re-reads.
__device__ __forceinline__ vec16 load16_stream(const void* p) {
    vec16 v;
    const uint32_t* q = reinterpret_cast<const uint32_t*>(p);
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    u4 t = __builtin_nontemporal_load(reinterpret_cast<const u4*>(q));
    v.w[0] = t.x; v.w[1] = t.y; v.w[2] = t.z; v.w[3] = t.w;
    return v;
}
__device__ __forceinline__ void store16_stream(void* p, const vec16& v) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    u4 t = {v.w[0], v.w[1], v.w[2], v.w[3]};
    __builtin_nontemporal_store(t, reinterpret_cast<u4*>(p));
}
// Non-temporal and written through the XCD's L2 (agent scope, "sc1 nt") instead of being left there
// dirty for a later write-back.  On a streaming copy: 5.0 TB/s with plain stores, 5.27 with "nt",
// 5.57 with "sc1 nt" (64 MiB of traffic); it helps the kernels that write to fresh memory (gather,
// QKV scatter, cache movers) and hurts the in-place norm and SwiGLU by 2 %, so it is a per-kernel
// choice.  The compiler has no builtin for this combination on a 16-byte vector, hence the
// one-instruction asm.  It is a vector-memory store like any other; the only thing the compiler does
// not see is its entry in the vector-memory counter, which can only make the waits it computes for
// later loads longer, never shorter (loads complete in order among themselves).
// The trailing s_nop is part of the instruction's contract on this hardware: a vector-memory store of
// more than 8 bytes reads its data registers one cycle after issue, and an instruction that rewrites
// them must not follow directly.  The compiler inserts that wait state for its own stores but cannot
// see into an asm block (without it, a second store whose address landed in the first store's data
// registers wrote address bits into the first one's output, a few elements per million).
__device__ __forceinline__ void store16_through(void* p, const vec16& v) {
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    u4 t = {v.w[0], v.w[1], v.w[2], v.w[3]};
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" : : "v"(p), "v"(t) : "memory");
}

// Store kinds selectable per kernel instantiation.
constexpr int kStorePlain = 0, kStoreStream = 1, kStoreThrough = 2;

template <int ST>
__device__ __forceinline__ void store16_sel(void* p, const vec16& v) {
    if (ST == kStoreThrough) store16_through(p, v);
    else if (ST == kStoreStream) store16_stream(p, v);
    else store16(p, v);
}

// Maps a store knob (0 = the kernel's own default, 1 = plain, 2 = non-temporal, 3 = non-temporal
// write-through) to a store kind.
inline int store_kind(int knob_value, int default_kind) {
    return knob_value == 1 ? kStorePlain : knob_value == 2 ? kStoreStream
         : knob_value == 3 ? kStoreThrough : default_kind;
}

// Element traits: how many elements a 16-byte vector holds and how to move between storage and fp32.
template <typename T>
struct Elem;

template <>
struct Elem<float> {
    static constexpr int kVec = 4;
    __device__ static __forceinline__ void unpack(const vec16& v, float* f) {
#pragma unroll
        for (int i = 0; i < 4; i++) f[i] = __uint_as_float(v.w[i]);
    }
    __device__ static __forceinline__ vec16 pack(const float* f) {
        vec16 v;
#pragma unroll
        for (int i = 0; i < 4; i++) v.w[i] = __float_as_uint(f[i]);
        return v;
    }
    __device__ static __forceinline__ float to_f32(float x) { return x; }
    __device__ static __forceinline__ float from_f32(float x) { return x; }
    __device__ static __forceinline__ float pinned(float x) { return x; }
    __device__ static __forceinline__ vec16 pack_pinned(const float* f) { return pack(f); }
    // x = a + b,  x += b,  y = g * x  on one vector, element by element in fp32
    __device__ static __forceinline__ void sum(const vec16& a, const vec16& b, float* x) {
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = __uint_as_float(a.w[i]) + __uint_as_float(b.w[i]);
    }
    __device__ static __forceinline__ void accumulate(const vec16& b, float* x) {
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] += __uint_as_float(b.w[i]);
    }
    __device__ static __forceinline__ void scale(const vec16& g, const float* x, float* y) {
#pragma unroll
        for (int i = 0; i < 4; i++) y[i] = __uint_as_float(g.w[i]) * x[i];
    }
};

template <>
struct Elem<__half> {
    static constexpr int kVec = 8;
    __device__ static __forceinline__ void unpack(const vec16& v, float* f) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            __half2 h = *reinterpret_cast<const __half2*>(&v.w[i]);
            float2 p = __half22float2(h);
            f[2 * i] = p.x;
            f[2 * i + 1] = p.y;
        }
    }
    // The fp32 value is pinned in a register before the conversion.  Without that the compiler may
    // merge the producing multiply-add with the conversion into one mixed-precision instruction
    // that rounds the exact product-sum straight to fp16; kernels would then differ from each other
    // (and from "fp32 arithmetic, one rounding of the fp32 result") on rounding ties.
    __device__ static __forceinline__ float pinned(float x) {
        asm volatile("" : "+v"(x));
        return x;
    }
    __device__ static __forceinline__ vec16 pack(const float* f) {
        vec16 v;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            __half2 h = __floats2half2_rn(pinned(f[2 * i]), pinned(f[2 * i + 1]));
            v.w[i] = *reinterpret_cast<const uint32_t*>(&h);
        }
        return v;
    }
    // For values that went through pinned() when they were produced and are used again afterwards:
    // pinning them a second time here would cost a register copy each.
    __device__ static __forceinline__ vec16 pack_pinned(const float* f) {
        vec16 v;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            __half2 h = __floats2half2_rn(f[2 * i], f[2 * i + 1]);
            v.w[i] = *reinterpret_cast<const uint32_t*>(&h);
        }
        return v;
    }
    __device__ static __forceinline__ float to_f32(__half x) { return __half2float(x); }
    __device__ static __forceinline__ __half from_f32(float x) { return __float2half_rn(pinned(x)); }
    // x = a + b,  x += b,  y = g * x  on one vector, element by element in fp32.  Written as
    // fma(half, 1, .) / fma(half, x, -0) with the constants hidden from the optimiser: the compiler
    // then emits one mixed-precision multiply-add that reads the fp16 operand directly, in place of
    // a conversion plus an add or multiply -- same value (the product with 1 and the sum with -0 are
    // exact), a third of the instructions.
    __device__ static __forceinline__ float lo(uint32_t w) {
        return __half2float(__ushort_as_half((unsigned short)(w & 0xffffu)));
    }
    __device__ static __forceinline__ float hi(uint32_t w) {
        return __half2float(__ushort_as_half((unsigned short)(w >> 16)));
    }
    __device__ static __forceinline__ float hidden_constant(float v) {
        asm volatile("" : "+v"(v));
        return v;
    }
    __device__ static __forceinline__ void sum(const vec16& a, const vec16& b, float* x) {
        const float one = hidden_constant(1.0f);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            x[2 * i] = __fmaf_rn(lo(a.w[i]), one, lo(b.w[i]));
            x[2 * i + 1] = __fmaf_rn(hi(a.w[i]), one, hi(b.w[i]));
        }
    }
    __device__ static __forceinline__ void accumulate(const vec16& b, float* x) {
        const float one = hidden_constant(1.0f);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            x[2 * i] = __fmaf_rn(lo(b.w[i]), one, x[2 * i]);
            x[2 * i + 1] = __fmaf_rn(hi(b.w[i]), one, x[2 * i + 1]);
        }
    }
    __device__ static __forceinline__ void scale(const vec16& g, const float* x, float* y) {
        const float negzero = hidden_constant(-0.0f);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            y[2 * i] = __fmaf_rn(lo(g.w[i]), x[2 * i], negzero);
            y[2 * i + 1] = __fmaf_rn(hi(g.w[i]), x[2 * i + 1], negzero);
        }
    }
};

// Unsigned division by a launch constant without the integer-divide expansion: q = floor(p / d) from
// one multiply-high and one correction step (exact for every 32-bit p).
struct FastDiv {
    unsigned d, m;  // m = floor(2^32 / d), saturated for d = 1
    __device__ __forceinline__ void divmod(unsigned p, unsigned& q, unsigned& r) const {
        q = __umulhi(p, m);
        r = p - q * d;
        if (r >= d) {
            q++;
            r -= d;
        }
    }
};

inline FastDiv make_fastdiv(unsigned d) {
    FastDiv f;
    f.d = d;
    f.m = d <= 1 ? 0xffffffffu : (unsigned)(0x100000000ull / d);
    return f;
}

// p[i] of an int32 array that no kernel of this library writes (token ids, sequence lengths), read through
// the constant address space so that a wave-uniform index takes the scalar path.  A __restrict__ kernel
// parameter gets that by itself; a pointer inside an argument struct, or one that has been named in an
// asm statement, does not: the compiler must then assume that the kernel's own stores could alias it,
// issues a vector load and waits for every earlier vector load -- the streamed rows -- before it looks at
// the value (fused KV append: 26.8 -> 26.05 us).
__device__ __forceinline__ int32_t read_only_i32(const int32_t* p, int i) {
    typedef const int32_t __attribute__((address_space(4)))* constant_ints;
    return reinterpret_cast<constant_ints>((unsigned long long)p)[i];
}

// DPP lane exchange inside the VALU (no LDS traffic).  `ctrl` is the DPP control word.
template <int ctrl>
__device__ __forceinline__ float dpp_mov(float x) {
    return __uint_as_float(
        __builtin_amdgcn_update_dpp(0u, __float_as_uint(x), ctrl, 0xf, 0xf, true));
}

// Sum over the 64 lanes of a wavefront; every lane receives the total.
// Four DPP steps fold each row of 16 lanes (quad swaps, then half-row and full-row mirrors), then
// the four row sums are read out as scalars and added as (r0 + r1) + (r2 + r3).  The association is
// the balanced binary tree over the lane index, lowest bit first: deterministic, and the same in
// every lane.  (Folding the rows with two DPP row broadcasts instead of the four read-outs gives the
// same tree in fewer instructions but a longer dependent chain, and measured 0.5 % slower.)
__device__ __forceinline__ float wave_sum(float x) {
    x += dpp_mov<0xB1>(x);   // quad_perm [1,0,3,2]
    x += dpp_mov<0x4E>(x);   // quad_perm [2,3,0,1]
    x += dpp_mov<0x141>(x);  // row_half_mirror
    x += dpp_mov<0x140>(x);  // row_mirror
    float a = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(x), 0));
    float b = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(x), 16));
    float c = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(x), 32));
    float d = __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(x), 48));
    return (a + b) + (c + d);
}

}  // namespace isp
