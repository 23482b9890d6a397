// a8.h — the activation format of the int8-MFMA GEMMs and the per-32 quantizer that writes it.
//
// Activations travel between kernels as "A8" blocks of 256 elements x 32 batch rows (10240 bytes):
//   codes  [8 groups][64 lanes][16 B]   lane (row m, half h) holds elements 16h..16h+15 of the group: the A operand of
//                                       v_mfma_i32_32x32x32_i8, so a wave load is one contiguous 1 KB read
//   scales [64 lanes][4] f32 @8192      lane (m, h) entry p: the scale of group 2p+h (maxabs/127, 1 for an all-zero group)
//   sums   [64 lanes][4] f32 @9216      lane (m, h) entry p: scale * sum of codes of group 2p+h
// exactly what linalg.QuantizeActQ(group 32) yields (codes and scales bit for bit; goinfer call sites decoder/weightmat.go:845-862,
// device twin backend/cuda/actgroup.cu:32-54 quantG32), laid out for the wave that consumes it.
#pragma once
#include "common.h"

#define RD_A8_BLOCK_BYTES 10240
#define RD_A8_SCALES 8192
#define RD_A8_SUMS 9216

// byte offset of the code of element k of batch row m
__device__ __forceinline__ size_t a8_code_offset(int m, int k) {
    const int g = k >> 5, e = k & 31;
    return (size_t)(g >> 3) * RD_A8_BLOCK_BYTES + ((g & 7) << 10) + ((((e >> 4) << 5) + m) << 4) + (e & 15);
}
// byte offset of the f32 scale of group g of batch row m (its sum sits RD_A8_SUMS - RD_A8_SCALES further on)
__device__ __forceinline__ size_t a8_scale_offset(int m, int g) {
    return (size_t)(g >> 3) * RD_A8_BLOCK_BYTES + RD_A8_SCALES + ((((((g & 1) << 5) + m) << 2) + ((g & 7) >> 1)) << 2);
}

// Per-32 quantization of one element per lane (an aligned half-wave is one group): goinfer's QuantizeActQ(group 32) with the CPU
// path's round-half-away. Returns the code; *sc = maxabs/127 (1 for an all-zero group) and *gsum = sc * sum(codes), the same on every lane of the group.
__device__ __forceinline__ int quant8_g32(float v, float *sc, float *gsum) {
    const float ma = wave_max32(fabsf(v));
    const float s = ma == 0.f ? 1.f : ma / 127.f; // an all-zero group: scale 1, codes 0 (linalg.QuantizeRowInt8's rule)
    const float inv = 1.f / s;
    float r = roundf(__fmul_rn(v, inv));
    r = fminf(127.f, fmaxf(-127.f, r));
    const int code = (int)r;
    *sc = s;
    *gsum = __fmul_rn(s, (float)wave_sum32_i(code));
    return code;
}
// The same when each lane holds four consecutive elements: a group is 8 consecutive lanes. Returns the four codes packed low byte first.
__device__ __forceinline__ uint32_t quant8_g32x4(float v0, float v1, float v2, float v3, float *sc, float *gsum) {
    float ma = fmaxf(fmaxf(fabsf(v0), fabsf(v1)), fmaxf(fabsf(v2), fabsf(v3)));
    ma = group_max8(ma);
    const float s = ma == 0.f ? 1.f : ma / 127.f;
    const float inv = 1.f / s;
    const int c0 = (int)fminf(127.f, fmaxf(-127.f, roundf(__fmul_rn(v0, inv)))), c1 = (int)fminf(127.f, fmaxf(-127.f, roundf(__fmul_rn(v1, inv))));
    const int c2 = (int)fminf(127.f, fmaxf(-127.f, roundf(__fmul_rn(v2, inv)))), c3 = (int)fminf(127.f, fmaxf(-127.f, roundf(__fmul_rn(v3, inv))));
    *sc = s;
    *gsum = __fmul_rn(s, (float)group_sum8_i(c0 + c1 + c2 + c3));
    return (uint32_t)(c0 & 255) | ((uint32_t)(c1 & 255) << 8) | ((uint32_t)(c2 & 255) << 16) | ((uint32_t)(c3 & 255) << 24);
}
// One scale for the whole row (goinfer's ActQuantGroup 0: linalg.QuantizeRowInt8, twin backend/cuda/kv8_store.cu:27-35): the
// four consecutive elements of a lane against the row's scale s = maxabs/127 (1 for an all-zero row), codes round-half-away.
// *gsum = s * sum of the codes of the lane's group of 32 (8 consecutive lanes), as the per-32 form stores it.
__device__ __forceinline__ float row_scale_of(float maxabs) { return maxabs == 0.f ? 1.f : maxabs / 127.f; }
__device__ __forceinline__ uint32_t quant8_rowx4(float v0, float v1, float v2, float v3, float s, float *gsum) {
    const float inv = 1.f / s;
    const int c0 = (int)fminf(127.f, fmaxf(-127.f, roundf(__fmul_rn(v0, inv)))), c1 = (int)fminf(127.f, fmaxf(-127.f, roundf(__fmul_rn(v1, inv))));
    const int c2 = (int)fminf(127.f, fmaxf(-127.f, roundf(__fmul_rn(v2, inv)))), c3 = (int)fminf(127.f, fmaxf(-127.f, roundf(__fmul_rn(v3, inv))));
    *gsum = __fmul_rn(s, (float)group_sum8_i(c0 + c1 + c2 + c3));
    return (uint32_t)(c0 & 255) | ((uint32_t)(c1 & 255) << 8) | ((uint32_t)(c2 & 255) << 16) | ((uint32_t)(c3 & 255) << 24);
}
// Stores four consecutive elements k0..k0+3 (k0 % 4 == 0) of batch row m and, from the group's first lane, its scale and sum.
__device__ __forceinline__ void a8_store4(uint8_t *__restrict__ A8, int m, int k0, uint32_t codes, float sc, float gsum) {
    *(uint32_t *)(A8 + a8_code_offset(m, k0)) = codes;
    if ((k0 & 31) == 0) {
        uint8_t *p = A8 + a8_scale_offset(m, k0 >> 5);
        *(float *)p = sc;
        *(float *)(p + (RD_A8_SUMS - RD_A8_SCALES)) = gsum;
    }
}

// ROW8: the same quantized activations as plain rows, for the kernels that walk one row's groups in order (the experts' GEMMs,
// which have a handful of rows each and run on the vector ALU): [32 rows][K] int8 codes, then [32][K/32] f32 scales, then
// [32][K/32] f32 scaled code sums. K % 32 == 0; 40 bytes per element column, the size of the A8 blocks of the same K.
__device__ __forceinline__ size_t row8_scales(int K) { return (size_t)32 * K; }
__device__ __forceinline__ size_t row8_sums(int K) { return (size_t)32 * K + (size_t)32 * (K >> 5) * 4; }
__device__ __forceinline__ void row8_store4(uint8_t *__restrict__ X, int K, int m, int k0, uint32_t codes, float sc, float gsum) {
    *(uint32_t *)(X + (size_t)m * K + k0) = codes;
    if ((k0 & 31) == 0) {
        *(float *)(X + row8_scales(K) + ((size_t)m * (K >> 5) + (k0 >> 5)) * 4) = sc;
        *(float *)(X + row8_sums(K) + ((size_t)m * (K >> 5) + (k0 >> 5)) * 4) = gsum;
    }
}
__device__ __forceinline__ void row8_store1(uint8_t *__restrict__ X, int K, int m, int k, int code, float sc, float gsum) {
    X[(size_t)m * K + k] = (uint8_t)code;
    if ((k & 31) == 0) {
        *(float *)(X + row8_scales(K) + ((size_t)m * (K >> 5) + (k >> 5)) * 4) = sc;
        *(float *)(X + row8_sums(K) + ((size_t)m * (K >> 5) + (k >> 5)) * 4) = gsum;
    }
}
