// common.h — shared device helpers for the gfx950 decode kernels (wave64, CDNA4).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

#define RD_WAVE 64

// Cross-lane exchanges on the VALU's data-parallel path (DPP) instead of the LDS crossbar: a few cycles each instead of
// an LDS round trip. Each returns, for every lane, the value of its partner lane: XOR1/XOR2 inside a quad, then the
// half-row and row mirrors (lane i <-> 7-i of its 8, lane i <-> 15-i of its 16) — partners in the other half, which is all
// a reduction needs once the lower levels are uniform — and lane i <-> i^16 through ds_swizzle.
#define RD_DPP_QUAD_XOR1 0xB1   // quad_perm:[1,0,3,2]
#define RD_DPP_QUAD_XOR2 0x4E   // quad_perm:[2,3,0,1]
#define RD_DPP_HALF_MIRROR 0x141 // row_half_mirror
#define RD_DPP_ROW_MIRROR 0x140  // row_mirror
// a*b rounded to f32 on its own. HIP's __fmul_rn is a plain product, which the compiler is free to contract with a following add
// into one FMA (one rounding instead of two); where the reference's arithmetic rounds the product first and an add follows, the
// product goes through here.
__device__ __forceinline__ float mul_rounded(float a, float b) {
#pragma clang fp contract(off)
    return a * b;
}

template <int CTRL> __device__ __forceinline__ int dpp_i(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true); }
template <int CTRL> __device__ __forceinline__ float dpp_f(float v) { return __int_as_float(dpp_i<CTRL>(__float_as_int(v))); }
__device__ __forceinline__ int swz_xor16_i(int v) { return __builtin_amdgcn_ds_swizzle(v, 0x401F); } // bit mode: and 0x1F, xor 0x10
__device__ __forceinline__ float swz_xor16_f(float v) { return __int_as_float(swz_xor16_i(__float_as_int(v))); }

// max / sum over each aligned group of 8, 16 or 32 lanes, delivered to every lane of the group
__device__ __forceinline__ float group_max8(float v) {
    v = fmaxf(v, dpp_f<RD_DPP_QUAD_XOR1>(v));
    v = fmaxf(v, dpp_f<RD_DPP_QUAD_XOR2>(v));
    return fmaxf(v, dpp_f<RD_DPP_HALF_MIRROR>(v));
}
__device__ __forceinline__ int group_sum8_i(int v) {
    v += dpp_i<RD_DPP_QUAD_XOR1>(v);
    v += dpp_i<RD_DPP_QUAD_XOR2>(v);
    return v + dpp_i<RD_DPP_HALF_MIRROR>(v);
}
__device__ __forceinline__ float group_max16(float v) {
    v = group_max8(v);
    return fmaxf(v, dpp_f<RD_DPP_ROW_MIRROR>(v));
}
__device__ __forceinline__ float wave_max32(float v) {
    v = group_max16(v);
    return fmaxf(v, swz_xor16_f(v));
}
__device__ __forceinline__ int wave_sum32_i(int v) {
    v = group_sum8_i(v);
    v += dpp_i<RD_DPP_ROW_MIRROR>(v);
    return v + swz_xor16_i(v);
}
__device__ __forceinline__ float wave_sum64(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ double wave_sum64_d(double v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}

// binary16 <- f32 with round-half-up on the dropped bits: goinfer's KV narrowing (internal/runtime/f16/f16.go:14-43).
__device__ __forceinline__ uint16_t f32_to_f16_half_up(float f) {
    uint32_t b = __float_as_uint(f);
    uint16_t sign = (uint16_t)((b >> 16) & 0x8000);
    int32_t e = (int32_t)((b >> 23) & 0xFF) - 112;
    uint32_t m = b & 0x7FFFFF;
    if (((b >> 23) & 0xFF) == 0xFF) return m ? (sign | 0x7E00) : (sign | 0x7C00);
    if (e >= 0x1F) return sign | 0x7C00;
    if (e <= 0) {
        if (e < -10) return sign;
        m |= 0x800000;
        uint32_t sh = (uint32_t)(14 - e);
        return sign | (uint16_t)((m + (1u << (sh - 1))) >> sh);
    }
    uint16_t half = sign | (uint16_t)(e << 10) | (uint16_t)(m >> 13);
    if (m & 0x1000) half++;
    return half;
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    half_t x;
    __builtin_memcpy(&x, &h, 2);
    return (float)x;
}
__device__ __forceinline__ uint16_t f16_to_bits(half_t x) {
    uint16_t h;
    __builtin_memcpy(&h, &x, 2);
    return h;
}

// Per-32 activation quantization of one element (goinfer: aikit QuantizeActQ group 32; backend/cuda/actgroup.cu:32-54,
// with the CPU path's round-half-away): the 32 lanes of an aligned half-wave hold one group.
// Returns the dequantized value code*scale; *gsum = scale * sum(codes) (the same on every lane of the group).
__device__ __forceinline__ float quant_g32(float v, float *gsum) {
    float ma = wave_max32(fabsf(v));
    float sc = ma / 127.f;
    float inv = sc > 0.f ? 1.f / sc : 0.f;
    float r = roundf(__fmul_rn(v, inv));
    r = fminf(127.f, fmaxf(-127.f, r));
    int code = (int)r;
    int s = wave_sum32_i(code);
    *gsum = __fmul_rn(sc, (float)s);
    return __fmul_rn((float)code, sc);
}

// silu(g) = f32(g64 / (1 + exp(-g64))), evaluated in f64 as goinfer does (decoder/rmsnorm.go:204-207). exp by range
// reduction and a degree-13 Taylor polynomial on |r| <= ln2/2 (remainder < 1e-17), the quotient by a Newton-refined
// reciprocal with one residual correction: the f64 value is within an ulp or two of the correctly rounded one, so the f32
// result differs from a libm evaluation only if it lies within ~1e-15 (relative) of an f32 rounding boundary. An order of
// magnitude fewer f64 instructions than exp() and an IEEE division. Huge magnitudes, inf and NaN take the library path.
__device__ __forceinline__ float silu_f64(float g) {
    const double g64 = (double)g;
    if (!(fabsf(g) <= 80.f)) return (float)(g64 / (1.0 + exp(-g64)));
    const double x = -g64;
    const double n = rint(x * 1.44269504088896338700e+00);
    double r = fma(n, -6.93147180369123816490e-01, x);
    r = fma(n, -1.90821492927058770002e-10, r);
    double p = 1.0 / 6227020800.0;
    p = fma(p, r, 1.0 / 479001600.0);
    p = fma(p, r, 1.0 / 39916800.0);
    p = fma(p, r, 1.0 / 3628800.0);
    p = fma(p, r, 1.0 / 362880.0);
    p = fma(p, r, 1.0 / 40320.0);
    p = fma(p, r, 1.0 / 5040.0);
    p = fma(p, r, 1.0 / 720.0);
    p = fma(p, r, 1.0 / 120.0);
    p = fma(p, r, 1.0 / 24.0);
    p = fma(p, r, 1.0 / 6.0);
    p = fma(p, r, 0.5);
    p = fma(p, r, 1.0);
    p = fma(p, r, 1.0);
    const double d = 1.0 + ldexp(p, (int)n);
    double y = __builtin_amdgcn_rcp(d);
    y = fma(fma(-d, y, 1.0), y, y);
    y = fma(fma(-d, y, 1.0), y, y);
    double q = g64 * y;
    q = fma(fma(-d, q, g64), y, q);
    return (float)q;
}

// The tanh-approximate GELU of Gemma's GeGLU (decoder/rmsnorm.go:229-234 geluTanh): f32(0.5 x (1 + tanh(c (x + 0.044715 x^3)))),
// every operation in f64 in goinfer's order, narrowed once. The products and sums are kept apart (no fused multiply-add): the
// reference rounds each of them.
__device__ __forceinline__ float gelu_tanh_f64(float g) {
    const double x = (double)g;
    const double cube = __dmul_rn(__dmul_rn(__dmul_rn(0.044715, x), x), x);
    const double inner = __dmul_rn(0.7978845608028654, __dadd_rn(x, cube));
    return (float)__dmul_rn(__dmul_rn(0.5, x), __dadd_rn(1.0, tanh(inner)));
}
// The gated FFN's activation: 0 = silu (SwiGLU), 1 = tanh-approximate GELU (GeGLU).
__device__ __forceinline__ float gate_act(float g, int act) { return act ? gelu_tanh_f64(g) : silu_f64(g); }
