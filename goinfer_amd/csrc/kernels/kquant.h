// kquant.h — the Q5_K and Q6_K lanes: bit-exact dequantization, re-tiling, and their traits for the int8-MFMA GEMMs of gemm8.h:
// the codes are 5- and 6-bit integers with integer sub-block scales, so the dot of a group is exact in int32 as it is for Q4_K
// (goinfer backend/cuda/actgroup.cu:85-205 rowsQ5K / rowsQ6K, :457-530 the kernels), and only the f32 fold's order differs from the oracle's.
//
// Formats (public ggml layouts; goinfer states the arithmetic at backend/cuda/actgroup.cu:77-137 for Q5_K and :139-205 for Q6_K):
//   Q5_K: 256 weights in 176 B: d f16 @0, dmin f16 @2, 12 B of 6-bit scales/mins @4 (as Q4_K), qh[32] @16, qs[128] @48.
//         Element 32j+l: nibble j&1 of qs[32*(j/2)+l], fifth bit = bit j of qh[l]; w = (d*sc_j)*q - dmin*m_j.
//   Q6_K: 256 weights in 210 B: ql[128] @0, qh[64] @128, 16 int8 scales @192, d f16 @208. In half n (128 weights), element
//         32g+l: nibble g/2 of ql[64n+32(g&1)+l], two high bits = bits 2g,2g+1 of qh[32n+l]; w = (d*sc[8n+2g+l/16])*(q-32).
#pragma once
#include "common.h"
#include "gemm8.h"
#include "q4k.h"

#define RD_Q5K_TILE_BYTES 5632 // 32 rows x 176 B: the Q4_K tile (512 B headers + 4 KB nibbles) + 1 KB of fifth bits
#define RD_Q6K_TILE_BYTES 7168 // 32 rows x 256 k: 1 KB of headers (per lane: 8 int8 scales, d) + 4 KB nibbles + 2 KB high bit pairs

__device__ __forceinline__ int q5k_code(const uint8_t *blk, int e) {
    int j = e >> 5, l = e & 31;
    int nib = (blk[48 + (j >> 1) * 32 + l] >> (4 * (j & 1))) & 15;
    return nib | (((blk[16 + l] >> j) & 1) << 4);
}
__device__ __forceinline__ int q6k_code(const uint8_t *blk, int e) { // unsigned 6-bit code, the weight is code-32
    int half = e >> 7, r = e & 127, g = r >> 5, l = r & 31;
    int nib = (blk[64 * half + 32 * (g & 1) + l] >> (4 * (g >> 1))) & 15;
    int hi = (blk[128 + 32 * half + l] >> (2 * g)) & 3;
    return nib | (hi << 4);
}

// One thread per weight, every product rounded separately as the CPU reference computes them.
extern "C" __global__ void rd_k_dequant_q5k(const uint8_t *__restrict__ blocks, float *__restrict__ out, long n_blocks) {
    long b = blockIdx.x;
    int t = threadIdx.x;
    if (b >= n_blocks) return;
    const uint8_t *blk = blocks + b * 176;
    int j = t >> 5, sc, m;
    q4k_scale_min(j, blk + 4, &sc, &m);
    float d = f16_bits_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
    float dmin = f16_bits_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
    float d1 = __fmul_rn(d, (float)sc), m1 = __fmul_rn(dmin, (float)m);
    out[b * 256 + t] = __fsub_rn(__fmul_rn(d1, (float)q5k_code(blk, t)), m1);
}
extern "C" __global__ void rd_k_dequant_q6k(const uint8_t *__restrict__ blocks, float *__restrict__ out, long n_blocks) {
    long b = blockIdx.x;
    int t = threadIdx.x;
    if (b >= n_blocks) return;
    const uint8_t *blk = blocks + b * 210;
    float d = f16_bits_to_f32((uint16_t)(blk[208] | (blk[209] << 8)));
    int sc = (int8_t)blk[192 + (t >> 4)];
    out[b * 256 + t] = __fmul_rn(__fmul_rn(d, (float)sc), (float)(q6k_code(blk, t) - 32));
}

// ---------------- Q5_K ----------------
// Tile of 32 rows x one super-block, 5632 B: the Q4_K tile of the same rows (32 headers of 16 B, then the four nibble planes, see
// rd_k_retile_q4k8) followed by one plane [64 lanes][16 B] of fifth bits: lane (row r, half h) holds qh[16h .. 16h+15] as the file
// has them, bit j of byte i the fifth bit of element 16h+i of sub-block j. The int8 operand of group g is nibble | bit << 4, 0..31;
// scales, minimum term and fold are Q4_K's (w = d*sc*q - dmin*m).
extern "C" __global__ __launch_bounds__(384) void rd_k_retile_q5k(const uint8_t *__restrict__ raw, uint8_t *__restrict__ tiled, int N, int nSB) {
    const int tile = blockIdx.x, sb = blockIdx.y, t = threadIdx.x; // 352 x 16 B
    if (t >= 352) return;
    uint8_t *dst = tiled + ((size_t)tile * nSB + sb) * RD_Q5K_TILE_BYTES;
    const uint4_t *src;
    if (t < 32) {
        src = (const uint4_t *)(raw + ((size_t)(tile * 32 + t) * nSB + sb) * 176);
    } else if (t < 288) {
        const int u = t - 32, p = u >> 6, lane = u & 63, r = lane & 31, h = lane >> 5;
        src = (const uint4_t *)(raw + ((size_t)(tile * 32 + r) * nSB + sb) * 176 + 48 + p * 32 + h * 16);
    } else {
        const int lane = t - 288, r = lane & 31, h = lane >> 5;
        src = (const uint4_t *)(raw + ((size_t)(tile * 32 + r) * nSB + sb) * 176 + 16 + h * 16);
    }
    *(uint4_t *)(dst + (size_t)t * 16) = *src;
}

struct Q5K8Tile {
    uint4_t hdr, q[4], hb;
};
struct Q5K8Traits {
    typedef Q5K8Tile Tile;
    static constexpr int TILE_BYTES = RD_Q5K_TILE_BYTES;
    static constexpr bool GEMV1 = false, INT_ACC = false; // one row runs on the matrix cores too: the same sums by construction
    static __device__ __forceinline__ void load(Tile &w, rd_rsrc_t r, int off, int lane) {
        w.hdr = buf_load16_nt(r, off + (lane & 31) * 16, 0);
#pragma unroll
        for (int c = 0; c < 4; c++) w.q[c] = buf_load16_nt(r, off + lane * 16, 512 + c * 1024);
        w.hb = buf_load16_nt(r, off + lane * 16, 4608);
    }
    template <int NR> static __device__ __forceinline__ void mma(float16_t &acc, const Tile &w, const A8Regs &a, const void *, int, int lane) {
        float dsc[4], ndm[4];
        Q4K8Tile hq;
        hq.hdr = w.hdr;
        Q4K8Traits::decode(hq, lane >> 5, dsc, ndm);
        const f32x32_t zero32 = {0.f};
        const i32x16_t zero16 = {0};
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const f32x32_t s2 = __builtin_amdgcn_mfma_f32_32x32x1f32(a.as[p], dsc[p], zero32, 0, 0, 0);
            const uint4_t raw = w.q[p];
            uint4_t lo, hi;
#pragma unroll
            for (int i = 0; i < 4; i++) { // sub-blocks 2p (low nibbles) and 2p+1 (high nibbles) with their fifth bits
                lo[i] = (raw[i] & 0x0F0F0F0Fu) | (((w.hb[i] >> (2 * p)) & 0x01010101u) << 4);
                hi[i] = ((raw[i] >> 4) & 0x0F0F0F0Fu) | (((w.hb[i] >> (2 * p + 1)) & 0x01010101u) << 4);
            }
            const i32x16_t d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[2 * p]), as_i32x4(lo), zero16, 0, 0, 0);
            const i32x16_t d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[2 * p + 1]), as_i32x4(hi), zero16, 0, 0, 0);
            RD_FOLD(acc, d0, s2, 0, NR)
            RD_FOLD(acc, d1, s2, 16, NR)
        }
#pragma unroll
        for (int p = 0; p < 4; p++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.asum[p], ndm[p], acc, 0, 0, 0);
    }
    static __device__ __forceinline__ void mma1(float16_t &, const Tile &, const A8Regs &, const void *, int, int) {}
    static __device__ __forceinline__ void finish(float16_t &, const void *, const uint8_t *, int, int) {}
};

// ---------------- Q6_K ----------------
// w = (d * sc_j) * (q - 32), one int8 scale per 16 weights: an activation group of 32 spans two sub-blocks, each half of the
// group with its own scale. In the int8 MFMA's operand order lane half h holds elements 16h..16h+15 of a group, which is
// exactly sub-block 2g+h: with the other half's codes set to zero one MFMA gives sub-block 2g's dot and a second one 2g+1's,
// exact int32 both, and each is folded with its own d * sc_j * aS_g (backend/cuda/actgroup.cu:139-205 rowsQ6K sums sc * idot per
// sub-block too; the oracle's sc_lo*idot_lo + sc_hi*idot_hi in integers is the same real number).
// Tile of 32 rows x one super-block, 7168 B: a header plane [64 lanes][16 B] (lane (row r, half h): the eight int8 scales of
// sub-blocks 2g+h, g = 0..7, then d as binary16), four nibble planes [64 lanes][16 B] (plane p, lane (r, h), byte i: element
// 16h+i of group 2p in the low nibble and of group 2p+1 in the high nibble), two planes of high bit pairs (plane x, word w of
// lane (r, h) = group 4x+w: byte k bits 2v..2v+1 = the pair of element 16h+4v+k). The code is stored as the 6-bit two's
// complement of q-32 (q ^ 32); put at the top of a byte it is the int8 4*(q-32), and the 1/4 rides in the scale.
extern "C" __global__ __launch_bounds__(448) void rd_k_retile_q6k(const uint8_t *__restrict__ raw, uint8_t *__restrict__ tiled, int N, int nSB) {
    const int tile = blockIdx.x, sb = blockIdx.y, t = threadIdx.x; // 448 x 16 B
    if (t >= 448) return;
    uint8_t *dst = tiled + ((size_t)tile * nSB + sb) * RD_Q6K_TILE_BYTES;
    const int u = t & 63, r = u & 31, h = u >> 5, plane = t >> 6;
    const uint8_t *blk = raw + ((size_t)(tile * 32 + r) * nSB + sb) * 210;
    uint8_t by[16];
#pragma unroll
    for (int i = 0; i < 16; i++) by[i] = 0;
    if (plane == 0) {
        for (int g = 0; g < 8; g++) by[g] = blk[192 + 2 * g + h];
        by[8] = blk[208], by[9] = blk[209];
    } else if (plane <= 4) {
        const int p = plane - 1;
        for (int i = 0; i < 16; i++) {
            const int lo = (q6k_code(blk, (2 * p) * 32 + 16 * h + i) ^ 32) & 15, hi = (q6k_code(blk, (2 * p + 1) * 32 + 16 * h + i) ^ 32) & 15;
            by[i] = (uint8_t)(lo | (hi << 4));
        }
    } else {
        const int x = plane - 5;
        for (int w = 0; w < 4; w++)
            for (int k = 0; k < 4; k++) {
                int b = 0;
                for (int v = 0; v < 4; v++) b |= (((q6k_code(blk, (4 * x + w) * 32 + 16 * h + 4 * v + k) ^ 32) >> 4) & 3) << (2 * v);
                by[4 * w + k] = (uint8_t)b;
            }
    }
    uint4_t v;
    __builtin_memcpy(&v, by, 16);
    *(uint4_t *)(dst + (size_t)t * 16) = v;
}

struct Q6K8Tile {
    uint4_t hdr, q[4], hb[2];
};
struct Q6K8Traits {
    typedef Q6K8Tile Tile;
    static constexpr int TILE_BYTES = RD_Q6K_TILE_BYTES;
    static constexpr bool GEMV1 = false, INT_ACC = false;
    static __device__ __forceinline__ void load(Tile &w, rd_rsrc_t r, int off, int lane) {
        w.hdr = buf_load16_nt(r, off + lane * 16, 0);
#pragma unroll
        for (int c = 0; c < 4; c++) w.q[c] = buf_load16_nt(r, off + lane * 16, 1024 + c * 1024);
        w.hb[0] = buf_load16_nt(r, off + lane * 16, 5120);
        w.hb[1] = buf_load16_nt(r, off + lane * 16, 6144);
    }
    template <int NR> static __device__ __forceinline__ void mma(float16_t &acc, const Tile &w, const A8Regs &a, const void *, int, int lane) {
        const bool upper = lane >= 32;
        const float d = f16_bits_to_f32((uint16_t)(w.hdr.z & 0xffffu)) * 0.25f; // the codes come out as 4 * (q - 32)
        const f32x32_t zero32 = {0.f};
        const i32x16_t zero16 = {0};
#pragma unroll
        for (int g = 0; g < 8; g++) {
            const int p = g >> 1;
            // this lane's sub-block (2g + its half) scale; the group's activation scale on both halves
            const int sci = (int)((g < 4 ? w.hdr.x : w.hdr.y) << (24 - 8 * (g & 3))) >> 24;
            float a_lo, a_hi;
            halves_f(a.as[p], a_lo, a_hi);
            const f32x32_t s2 = __builtin_amdgcn_mfma_f32_32x32x1f32((g & 1) ? a_hi : a_lo, __fmul_rn(d, (float)sci), zero32, 0, 0, 0);
            const uint4_t raw = w.q[p];
            const uint32_t hw = w.hb[g >> 2][g & 3];
            uint4_t c, cl, ch;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t nib = (g & 1) ? (raw[i] >> 2) & 0x3C3C3C3Cu : (raw[i] << 2) & 0x3C3C3C3Cu;
                c[i] = nib | ((hw << (6 - 2 * i)) & 0xC0C0C0C0u);
                cl[i] = upper ? 0u : c[i], ch[i] = upper ? c[i] : 0u;
            }
            const i32x16_t d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[g]), as_i32x4(cl), zero16, 0, 0, 0);
            const i32x16_t d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[g]), as_i32x4(ch), zero16, 0, 0, 0);
            RD_FOLD(acc, d0, s2, 0, NR)
            RD_FOLD(acc, d1, s2, 16, NR)
        }
    }
    static __device__ __forceinline__ void mma1(float16_t &, const Tile &, const A8Regs &, const void *, int, int) {}
    static __device__ __forceinline__ void finish(float16_t &, const void *, const uint8_t *, int, int) {}
};

RD_GEMM8_KERNEL(rd_k_gemm8_q5k_kw2, Q5K8Traits, 2, 2)
RD_GEMM8_KERNEL(rd_k_gemm8_q5k_kw4, Q5K8Traits, 4, 1)
RD_GEMM8_KERNEL(rd_k_gemm8_q5k_kw8, Q5K8Traits, 8, 1)
RD_GEMM8_KERNEL(rd_k_gemm8_q6k_kw2, Q6K8Traits, 2, 2)
RD_GEMM8_KERNEL(rd_k_gemm8_q6k_kw4, Q6K8Traits, 4, 1)
RD_GEMM8_KERNEL(rd_k_gemm8_q6k_kw8, Q6K8Traits, 8, 1)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_q5k_qkv_kw2, Q5K8Traits, 2)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_q5k_qkv_kw4, Q5K8Traits, 4)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_q5k_qkv_kw8, Q5K8Traits, 8)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_q6k_qkv_kw2, Q6K8Traits, 2)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_q6k_qkv_kw4, Q6K8Traits, 4)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_q6k_qkv_kw8, Q6K8Traits, 8)
