// kquant.h — the Q5_K and Q6_K lanes: bit-exact dequantization, re-tiling, and dequant-GEMMs on the shared skeleton.
//
// Formats (public ggml layouts; goinfer states the arithmetic at backend/cuda/actgroup.cu:77-137 for Q5_K and :139-205 for Q6_K):
//   Q5_K: 256 weights in 176 B: d f16 @0, dmin f16 @2, 12 B of 6-bit scales/mins @4 (as Q4_K), qh[32] @16, qs[128] @48.
//         Element 32j+l: nibble j&1 of qs[32*(j/2)+l], fifth bit = bit j of qh[l]; w = (d*sc_j)*q - dmin*m_j.
//   Q6_K: 256 weights in 210 B: ql[128] @0, qh[64] @128, 16 int8 scales @192, d f16 @208. In half n (128 weights), element
//         32g+l: nibble g/2 of ql[64n+32(g&1)+l], two high bits = bits 2g,2g+1 of qh[32n+l]; w = (d*sc[8n+2g+l/16])*(q-32).
#pragma once
#include "common.h"
#include "gemm.h"
#include "q4k.h"

#define RD_Q5K_TILE_BYTES 5632 // 32 rows x 176 B: the Q4_K tile (512 B headers + 4 KB nibbles) + 1 KB of fifth bits
#define RD_Q6K_TILE_BYTES 3456 // 32 rows x 128 k: 384 B of headers (8 int8 scales, d, pad) + 2 KB nibbles + 1 KB high bit pairs

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
// Tile = the Q4_K tile of the same rows (headers; nibble planes in raw byte order) followed by one plane [64 lanes][16 B]
// of fifth bits arranged for the unpack: word w of lane (row r, half h) serves MFMA steps 4w..4w+3. Step s reads nibble
// bytes l0..l0+3 (l0 = 4*(s%8)) of pass p = 2h + s/8, i.e. sub-blocks 2p (low nibbles) and 2p+1 (high nibbles). Its four
// half2 extractions are e0 = (2p; l0, l0+2), e1 = (2p+1; l0, l0+2), e2 = (2p; l0+1, l0+3), e3 = (2p+1; l0+1, l0+3); each
// needs its two fifth bits at bit 4|20 (e0, e2: the code sits in mantissa bits 0-4) or 8|24 (e1, e3: bits 4-8). With the
// word shifted by k = -4, -2, 4, 6 for s%4 = 0..3, e0 and e1 sit in place and one more shift by 1 places e2 and e3.
__device__ __forceinline__ int q5k_shift(int i) { return i == 0 ? -4 : (i == 1 ? -2 : (i == 2 ? 4 : 6)); }

extern "C" __global__ __launch_bounds__(384) void rd_k_retile_q5k(const uint8_t *__restrict__ raw, uint8_t *__restrict__ tiled, int N, int nSB) {
    int tile = blockIdx.x, sb = blockIdx.y;
    int t = threadIdx.x; // 0..351: 352 x 16 B = 5632 B
    if (t >= 352) return;
    uint8_t *dst = tiled + ((size_t)tile * nSB + sb) * RD_Q5K_TILE_BYTES;
    uint4_t v;
    if (t < 32) {
        v = *(const uint4_t *)(raw + ((size_t)(tile * 32 + t) * nSB + sb) * 176);
    } else if (t < 288) {
        int u = t - 32, c = u >> 6, lane = u & 63, r = lane & 31, h = lane >> 5;
        v = *(const uint4_t *)(raw + ((size_t)(tile * 32 + r) * nSB + sb) * 176 + 48 + h * 64 + c * 16);
    } else {
        int lane = t - 288, r = lane & 31, h = lane >> 5;
        const uint8_t *qh = raw + ((size_t)(tile * 32 + r) * nSB + sb) * 176 + 16;
        for (int w = 0; w < 4; w++) {
            uint32_t word = 0;
            for (int i = 0; i < 4; i++) {
                int s = 4 * w + i, p = 2 * h + (s >> 3), l0 = 4 * (s & 7), k = q5k_shift(i);
                for (int e = 0; e < 4; e++) {
                    int j = 2 * p + (e & 1), la = l0 + (e >> 1), lb = la + 2;
                    int pos = ((e & 1) ? 8 : 4) + (e >> 1) + k;
                    word |= (uint32_t)((qh[la] >> j) & 1) << pos;
                    word |= (uint32_t)((qh[lb] >> j) & 1) << (pos + 16);
                }
            }
            v[w] = word;
        }
    }
    *(uint4_t *)(dst + (size_t)t * 16) = v;
}

struct Q5KTile {
    uint4_t hdr, q[4], hb;
};

struct Q5KTraits {
    typedef Q5KTile Tile;
    static constexpr int TILE_BYTES = RD_Q5K_TILE_BYTES;
    static constexpr int PANEL_VECS = RD_Q4K_PANEL_BYTES / 16;
    static constexpr int PRODUCER_DEPTH = 2;
    static __device__ __forceinline__ void load(Tile &w, const uint8_t *__restrict__ p, int lane) {
        w.hdr = __builtin_nontemporal_load((const uint4_t *)(p + (lane & 31) * 16));
#pragma unroll
        for (int c = 0; c < 4; c++) w.q[c] = __builtin_nontemporal_load((const uint4_t *)(p + 512 + c * 1024 + lane * 16));
        w.hb = __builtin_nontemporal_load((const uint4_t *)(p + 4608 + lane * 16));
    }
    // As the Q4_K tile product with five-bit codes: 0x6400|q = 1024+q, 0x5400|(q<<4) = 64+q, centred at 16:
    // w = (q-16)*dsc + (16*dsc - dmin*m), the exact remainder of the fma constant folded into the offset step.
    static __device__ __forceinline__ void mma(float16_t &acc, const Tile &w, const uint4_t *__restrict__ panel, int lane) {
        const int h = lane >> 5;
        const uint32_t mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic_lo = 0x64006400u, magic_hi = 0x54005400u;
        const uint32_t bit_lo = 0x00100010u, bit_hi = 0x01000100u;
        uint32_t y = w.hdr.y, z = w.hdr.z, x = w.hdr.w;
        half2_t dd;
        uint32_t hx = w.hdr.x;
        __builtin_memcpy(&dd, &hx, 4);
        float d = (float)dd.x, dmin = (float)dd.y;
        half2_t DSC[4], C0[4];
        half_t off[4];
#pragma unroll
        for (int jj = 0; jj < 4; jj++) {
            int sc_lo = (y >> (8 * jj)) & 63, m_lo = (z >> (8 * jj)) & 63;
            int sc_hi = ((x >> (8 * jj)) & 15) | (((y >> (8 * jj + 6)) & 3) << 4);
            int m_hi = ((x >> (8 * jj + 4)) & 15) | (((z >> (8 * jj + 6)) & 3) << 4);
            int sc = h ? sc_hi : sc_lo, m = h ? m_hi : m_lo;
            float dsc32 = d * (float)sc;
            half_t dsc = (half_t)dsc32;
            float dscf = (float)dsc;
            const float bias = (jj & 1) ? 80.f : 1040.f;
            half_t c = (half_t)(-bias * dscf);
            float delta = (float)c + bias * dscf;
            DSC[jj] = (half2_t){dsc, dsc};
            C0[jj] = (half2_t){c, c};
            off[jj] = (half_t)(16.f * dsc32 - delta - dmin * (float)m);
        }
#pragma unroll
        for (int s = 0; s < 16; s++) {
            uint32_t wd = w.q[s >> 2][s & 3], H = w.hb[s >> 2];
            const int pp = s >> 3, k = q5k_shift(s & 3);
            uint32_t t8 = wd >> 8, Hs = k < 0 ? H << (-k) : H >> k, H1 = Hs >> 1;
            uint32_t u0 = and_or(Hs, bit_lo, and_or(wd, mask_lo, magic_lo)), u1 = and_or(Hs, bit_hi, and_or(wd, mask_hi, magic_hi));
            uint32_t u2 = and_or(H1, bit_lo, and_or(t8, mask_lo, magic_lo)), u3 = and_or(H1, bit_hi, and_or(t8, mask_hi, magic_hi));
            half2_t v0, v1, v2, v3;
            __builtin_memcpy(&v0, &u0, 4);
            __builtin_memcpy(&v1, &u1, 4);
            __builtin_memcpy(&v2, &u2, 4);
            __builtin_memcpy(&v3, &u3, 4);
            v0 = __builtin_elementwise_fma(v0, DSC[2 * pp], C0[2 * pp]);
            v1 = __builtin_elementwise_fma(v1, DSC[2 * pp + 1], C0[2 * pp + 1]);
            v2 = __builtin_elementwise_fma(v2, DSC[2 * pp], C0[2 * pp]);
            v3 = __builtin_elementwise_fma(v3, DSC[2 * pp + 1], C0[2 * pp + 1]);
            half8_t b = {v0.x, v0.y, v1.x, v1.y, v2.x, v2.y, v3.x, v3.y};
            half8_t a;
            uint4_t av = panel[s * 64 + lane];
            __builtin_memcpy(&a, &av, 16);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc, 0, 0, 0);
        }
        {
            half8_t b = {off[0], off[1], off[2], off[3], (half_t)0, (half_t)0, (half_t)0, (half_t)0};
            half8_t a;
            uint4_t av = panel[16 * 64 + lane];
            __builtin_memcpy(&a, &av, 16);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc, 0, 0, 0);
        }
    }
    static __device__ __forceinline__ void finish(float16_t &, const void *, int, int) {}
};

extern "C" __global__ __launch_bounds__(320) void rd_k_gemm_q5k(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ Xp,
                                                                 float *__restrict__ P, int N, int nSB, int sbPerSplit, int M, int ldP) {
    __shared__ uint4_t lds[2 * RD_Q4K_PANEL_BYTES / 16];
    gemm_body<Q5KTraits, 4, 1, 3>(Wt, nullptr, Xp, P, N, nSB, sbPerSplit, M, ldP, lds);
}

// ---------------- Q6_K ----------------
// K-blocks of 128 (one half of a super-block) against plain panels, so MFMA step s of a block is exactly sub-block s of
// the half (16 weights, one int8 scale). Tile of 32 rows: [32 rows][12 B] = 8 scales, d, 2 B pad; then planes
// [64 lanes][16 B]: nibble words of steps 0-3, of steps 4-7, and the high bit pairs. For lane (row r, half h), step s, the
// eight weights k = 16s+8h+i (i = 0..7) go to slots i of the B fragment: nibble i sits at bit [0,16,4,20,8,24,12,28][i] of
// the step's word, so the four half2 extractions are e0 = slots 0,1, e1 = 2,3 (bits 4-7|20-23), e2 = 4,5 and e3 = 6,7 after
// a shift by 8. High-bit word j serves steps 2j (shift k = -4) and 2j+1 (k = +4): after the shift the pairs of e0 sit at
// bits 4-5|20-21, of e1 at 8-9|24-25, and two bits further up those of e2 and e3.
extern "C" __global__ __launch_bounds__(256) void rd_k_retile_q6k(const uint8_t *__restrict__ raw, uint8_t *__restrict__ tiled, int N, int nSB) {
    int tile = blockIdx.x, kb = blockIdx.y, sb = kb >> 1, half = kb & 1;
    int t = threadIdx.x;
    uint8_t *dst = tiled + ((size_t)tile * (2 * nSB) + kb) * RD_Q6K_TILE_BYTES;
    if (t < 32) {
        const uint8_t *blk = raw + ((size_t)(tile * 32 + t) * nSB + sb) * 210;
        uint32_t a = 0, b = 0;
        for (int i = 0; i < 4; i++) a |= (uint32_t)blk[192 + 8 * half + i] << (8 * i), b |= (uint32_t)blk[192 + 8 * half + 4 + i] << (8 * i);
        uint32_t *o = (uint32_t *)(dst + t * 12);
        o[0] = a, o[1] = b, o[2] = (uint32_t)blk[208] | ((uint32_t)blk[209] << 8);
    } else if (t >= 64) {
        int u = t - 64, c = u >> 6, lane = u & 63, r = lane & 31, h = lane >> 5;
        const uint8_t *blk = raw + ((size_t)(tile * 32 + r) * nSB + sb) * 210;
        uint4_t v;
        for (int w = 0; w < 4; w++) {
            uint32_t word = 0;
            if (c < 2) {
                int s = 4 * c + w;
                for (int i = 0; i < 8; i++) {
                    int code = q6k_code(blk, 128 * half + 16 * s + 8 * h + i);
                    word |= (uint32_t)(code & 15) << (4 * ((i >> 1) + 4 * (i & 1)));
                }
            } else {
                for (int par = 0; par < 2; par++) {
                    int s = 2 * w + par, k = par ? 4 : -4;
                    for (int e = 0; e < 4; e++) {
                        int pos = ((e & 1) ? 8 : 4) + 2 * (e >> 1) + k;
                        int ca = q6k_code(blk, 128 * half + 16 * s + 8 * h + 2 * e), cb = q6k_code(blk, 128 * half + 16 * s + 8 * h + 2 * e + 1);
                        word |= (uint32_t)(ca >> 4) << pos;
                        word |= (uint32_t)(cb >> 4) << (pos + 16);
                    }
                }
            }
            v[w] = word;
        }
        *(uint4_t *)(dst + 384 + (size_t)u * 16) = v;
    }
}

struct Q6KTile {
    uint32_t sc0, sc1, d;
    uint4_t q[2], hb;
};

struct Q6KTraits {
    typedef Q6KTile Tile;
    static constexpr int TILE_BYTES = RD_Q6K_TILE_BYTES;
    static constexpr int PANEL_VECS = RD_LIN_PANEL_BYTES / 16;
    static constexpr int PRODUCER_DEPTH = 4;
    static __device__ __forceinline__ void load(Tile &w, const uint8_t *__restrict__ p, int lane) {
        const uint32_t *hp = (const uint32_t *)(p + (lane & 31) * 12);
        w.sc0 = __builtin_nontemporal_load(hp);
        w.sc1 = __builtin_nontemporal_load(hp + 1);
        w.d = __builtin_nontemporal_load(hp + 2);
        w.q[0] = __builtin_nontemporal_load((const uint4_t *)(p + 384 + lane * 16));
        w.q[1] = __builtin_nontemporal_load((const uint4_t *)(p + 384 + 1024 + lane * 16));
        w.hb = __builtin_nontemporal_load((const uint4_t *)(p + 384 + 2048 + lane * 16));
    }
    // code -> f16 exactly (0x6400|q = 1024+q, 0x5400|(q<<4) = 64+q), minus 1024+32 or 64+32 exactly, times f16(d*sc): each
    // weight (q-32)*dsc is rounded once.
    static __device__ __forceinline__ void mma(float16_t &acc, const Tile &w, const uint4_t *__restrict__ panel, int lane) {
        const uint32_t mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic_lo = 0x64006400u, magic_hi = 0x54005400u;
        const uint32_t pair_lo = 0x00300030u, pair_hi = 0x03000300u;
        const half2_t o_lo = {(half_t)(-1056.f), (half_t)(-1056.f)}, o_hi = {(half_t)(-96.f), (half_t)(-96.f)};
        half2_t dd;
        uint32_t dw = w.d;
        __builtin_memcpy(&dd, &dw, 4);
        const float d = (float)dd.x;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            uint32_t scw = s < 4 ? w.sc0 : w.sc1;
            int sci = (int)(scw << (24 - 8 * (s & 3))) >> 24;
            half_t dsc = (half_t)(d * (float)sci);
            half2_t sc = {dsc, dsc};
            uint32_t wd = w.q[s >> 2][s & 3], H = w.hb[s >> 1];
            uint32_t t8 = wd >> 8, Hs = (s & 1) ? H >> 4 : H << 4, H2 = Hs >> 2;
            uint32_t u0 = and_or(Hs, pair_lo, and_or(wd, mask_lo, magic_lo)), u1 = and_or(Hs, pair_hi, and_or(wd, mask_hi, magic_hi));
            uint32_t u2 = and_or(H2, pair_lo, and_or(t8, mask_lo, magic_lo)), u3 = and_or(H2, pair_hi, and_or(t8, mask_hi, magic_hi));
            half2_t v0, v1, v2, v3;
            __builtin_memcpy(&v0, &u0, 4);
            __builtin_memcpy(&v1, &u1, 4);
            __builtin_memcpy(&v2, &u2, 4);
            __builtin_memcpy(&v3, &u3, 4);
            v0 = (v0 + o_lo) * sc, v1 = (v1 + o_hi) * sc, v2 = (v2 + o_lo) * sc, v3 = (v3 + o_hi) * sc;
            half8_t b = {v0.x, v0.y, v1.x, v1.y, v2.x, v2.y, v3.x, v3.y};
            half8_t a;
            uint4_t av = panel[s * 64 + lane];
            __builtin_memcpy(&a, &av, 16);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc, 0, 0, 0);
        }
    }
    static __device__ __forceinline__ void finish(float16_t &, const void *, int, int) {}
};

extern "C" __global__ __launch_bounds__(320) void rd_k_gemm_q6k(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ Xp,
                                                                 float *__restrict__ P, int N, int nKB, int kbPerSplit, int M, int ldP) {
    __shared__ uint4_t lds[2 * RD_LIN_PANEL_BYTES / 16];
    gemm_body<Q6KTraits, 4, 1, 3>(Wt, nullptr, Xp, P, N, nKB, kbPerSplit, M, ldP, lds);
}
