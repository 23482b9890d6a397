// q4k.h — the Q4_K format: scale/minimum unpacking and the bit-exact dequantization kernel (the GEMM is in gemm8.h).
//
// Format (goinfer decoder/gguf.go:1508-1537, backend/cuda/actgroup.cu:56-75): a super-block is 256 weights in 144 bytes:
// d f16 @0, dmin f16 @2, 12 bytes of packed 6-bit scales/mins @4, 128 bytes of nibbles @16; w = d*sc_j*q - dmin*m_j.
#pragma once
#include "common.h"

__device__ __forceinline__ void q4k_scale_min(int j, const uint8_t *q, int *sc, int *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (q[j + 4] & 15) | ((q[j - 4] >> 6) << 4);
        *m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
    }
}

// One thread per weight. Bit-exact: (d*sc) and (dmin*m) are rounded products, then (d*sc)*q and the subtraction are
// rounded separately (no fused multiply-add), as the CPU reference computes them.
extern "C" __global__ void rd_k_dequant_q4k(const uint8_t *__restrict__ blocks, float *__restrict__ out, long n_blocks) {
    long b = blockIdx.x;
    int t = threadIdx.x; // 0..255
    if (b >= n_blocks) return;
    const uint8_t *blk = blocks + b * 144;
    int j = t >> 5, l = t & 31, sc, m;
    q4k_scale_min(j, blk + 4, &sc, &m);
    float d = f16_bits_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
    float dmin = f16_bits_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
    int q = (blk[16 + (j >> 1) * 32 + l] >> (4 * (j & 1))) & 15;
    float d1 = __fmul_rn(d, (float)sc), m1 = __fmul_rn(dmin, (float)m);
    out[b * 256 + t] = __fsub_rn(__fmul_rn(d1, (float)q), m1);
}

// (a & b) | c in one VALU op. Both constants must sit in VGPRs: a VOP3 instruction on this ISA takes no literal and at
// most one scalar operand, so the compiler otherwise emits v_and + v_or.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t b, uint32_t c) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
