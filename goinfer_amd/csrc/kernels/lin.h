// lin.h — int8 per-row (W8A8) and int4 group-32 (W4A8) weight kinds on the shared GEMM skeleton.
// Both use 128-wide K-blocks and "plain" activation panels (8 MFMA steps of 16 k).
#pragma once
#include "common.h"
#include "gemm.h"
#include "q4k.h"

// ---------------- W8A8: int8 codes, one f32 scale per row (goinfer WeightMat.Int8, decoder/weightmat.go:931) ----------------
// Tile of 32 rows x 128 k = 4096 B as 4 planes [64 lanes][16 B]; lane (row r, half h) plane c holds codes
// k = (2c)*16+h*8 .. +8 then k = (2c+1)*16+h*8 .. +8: steps 2c and 2c+1.
extern "C" __global__ __launch_bounds__(256) void rd_k_retile_w8a8(const uint8_t *__restrict__ raw, uint8_t *__restrict__ tiled, int N, int K) {
    int tile = blockIdx.x, kb = blockIdx.y, t = threadIdx.x;
    int c = t >> 6, lane = t & 63, r = lane & 31, h = lane >> 5;
    const uint8_t *row = raw + (size_t)(tile * 32 + r) * K + kb * 128;
    uint2_t a = *(const uint2_t *)(row + (2 * c) * 16 + h * 8), b = *(const uint2_t *)(row + (2 * c + 1) * 16 + h * 8);
    uint4_t v = {a.x, a.y, b.x, b.y};
    *(uint4_t *)(tiled + ((size_t)tile * (K / 128) + kb) * 4096 + (size_t)t * 16) = v;
}

struct W8Tile {
    uint4_t q[4];
};

struct W8Traits {
    typedef W8Tile Tile;
    static constexpr int TILE_BYTES = 4096;
    static constexpr int PANEL_VECS = RD_LIN_PANEL_BYTES / 16;
    static constexpr int PRODUCER_DEPTH = 4; // 8 KB panels, short K-blocks: more of them in flight
    static __device__ __forceinline__ void load(Tile &w, const uint8_t *__restrict__ p, int lane) {
#pragma unroll
        for (int c = 0; c < 4; c++) w.q[c] = __builtin_nontemporal_load((const uint4_t *)(p + c * 1024 + lane * 16));
    }
    // int8 -> f16 exactly: (b ^ 0x80) is b+128 unsigned; byte-permute it under 0x64 gives 1024+128+b; subtract 1152.
    static __device__ __forceinline__ void mma(float16_t &acc, const Tile &w, const uint4_t *__restrict__ panel, int lane) {
        const half2_t off = {(half_t)(-1152.f), (half_t)(-1152.f)};
#pragma unroll
        for (int s = 0; s < 8; s++) {
            uint32_t w0 = w.q[s >> 1][(s & 1) * 2] ^ 0x80808080u, w1 = w.q[s >> 1][(s & 1) * 2 + 1] ^ 0x80808080u;
            uint32_t u0 = __builtin_amdgcn_perm(0x64646464u, w0, 0x04010400u), u1 = __builtin_amdgcn_perm(0x64646464u, w0, 0x04030402u);
            uint32_t u2 = __builtin_amdgcn_perm(0x64646464u, w1, 0x04010400u), u3 = __builtin_amdgcn_perm(0x64646464u, w1, 0x04030402u);
            half2_t v0, v1, v2, v3;
            __builtin_memcpy(&v0, &u0, 4);
            __builtin_memcpy(&v1, &u1, 4);
            __builtin_memcpy(&v2, &u2, 4);
            __builtin_memcpy(&v3, &u3, 4);
            v0 += off, v1 += off, v2 += off, v3 += off;
            half8_t b = {v0.x, v0.y, v1.x, v1.y, v2.x, v2.y, v3.x, v3.y};
            half8_t a;
            uint4_t av = panel[s * 64 + lane];
            __builtin_memcpy(&a, &av, 16);
            acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc, 0, 0, 0);
        }
    }
    // the per-row weight scale multiplies the finished sum (backend/cuda/actgroup.cu:432)
    static __device__ __forceinline__ void finish(float16_t &acc, const void *aux, int tile, int lane) {
        float ws = ((const float *)aux)[tile * 32 + (lane & 31)];
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = __fmul_rn(acc[r], ws);
    }
};

extern "C" __global__ __launch_bounds__(320) void rd_k_gemm_w8a8(const uint8_t *__restrict__ Wt, const float *__restrict__ wscale,
                                                                  const uint8_t *__restrict__ Xp, float *__restrict__ P, int N, int nKB,
                                                                  int kbPerSplit, int M, int ldP) {
    __shared__ uint4_t lds[2 * RD_LIN_PANEL_BYTES / 16];
    gemm_body<W8Traits, 4, 1, 3>(Wt, wscale, Xp, P, N, nKB, kbPerSplit, M, ldP, lds);
}

// ---------------- W4A8: canonical int4 nibbles (value nib-8), binary16 scale per 32 (decoder/weightmat.go:160-178) ----------------
// Tile of 32 rows x 128 k = 2304 B: [32 rows][4 f16 scales] (256 B) then 2 planes [64 lanes][16 B]; lane (r,h) plane c word i is
// step s=4c+i: the 8 weights k = s*16+h*8 .. +8 (4 raw bytes). Unpacked slot order is [0,4,1,5,2,6,3,7]; the LIN4 panels match it.
extern "C" __global__ __launch_bounds__(320) void rd_k_retile_w4a8(const uint8_t *__restrict__ nib, const uint16_t *__restrict__ s16,
                                                                    uint8_t *__restrict__ tiled, int N, int K) {
    int tile = blockIdx.x, kb = blockIdx.y, t = threadIdx.x;
    uint8_t *dst = tiled + ((size_t)tile * (K / 128) + kb) * 2304;
    if (t < 32) {
        const uint16_t *s = s16 + (size_t)(tile * 32 + t) * (K / 32) + kb * 4;
        uint2_t v = {(uint32_t)s[0] | ((uint32_t)s[1] << 16), (uint32_t)s[2] | ((uint32_t)s[3] << 16)};
        *(uint2_t *)(dst + t * 8) = v;
    } else if (t >= 64 && t < 64 + 128) {
        int u = t - 64, c = u >> 6, lane = u & 63, r = lane & 31, h = lane >> 5;
        const uint8_t *row = nib + (size_t)(tile * 32 + r) * (K / 2) + kb * 64;
        uint4_t v;
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = *(const uint32_t *)(row + ((4 * c + i) * 16 + h * 8) / 2);
        *(uint4_t *)(dst + 256 + (size_t)u * 16) = v;
    }
}

struct W4Tile {
    uint2_t sc;
    uint4_t q[2];
};

struct W4Traits {
    typedef W4Tile Tile;
    static constexpr int TILE_BYTES = 2304;
    static constexpr int PANEL_VECS = RD_LIN_PANEL_BYTES / 16;
    static constexpr int PRODUCER_DEPTH = 4; // 8 KB panels, short K-blocks: more of them in flight
    static __device__ __forceinline__ void load(Tile &w, const uint8_t *__restrict__ p, int lane) {
        w.sc = __builtin_nontemporal_load((const uint2_t *)(p + (lane & 31) * 8));
        w.q[0] = __builtin_nontemporal_load((const uint4_t *)(p + 256 + lane * 16));
        w.q[1] = __builtin_nontemporal_load((const uint4_t *)(p + 256 + 1024 + lane * 16));
    }
    static __device__ __forceinline__ void mma(float16_t &acc, const Tile &w, const uint4_t *__restrict__ panel, int lane) {
        const half2_t o_lo = {(half_t)(-1032.f), (half_t)(-1032.f)}, o_hi = {(half_t)(-72.f), (half_t)(-72.f)};
        const uint32_t mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic_lo = 0x64006400u, magic_hi = 0x54005400u;
        half2_t s01, s23;
        uint32_t a0 = w.sc.x, a1 = w.sc.y;
        __builtin_memcpy(&s01, &a0, 4);
        __builtin_memcpy(&s23, &a1, 4);
        half_t gs[4] = {s01.x, s01.y, s23.x, s23.y};
#pragma unroll
        for (int s = 0; s < 8; s++) {
            uint32_t wd = w.q[s >> 2][s & 3], t8 = wd >> 8;
            half2_t sc = {gs[s >> 1], gs[s >> 1]};
            uint32_t u0 = and_or(wd, mask_lo, magic_lo), u1 = and_or(wd, mask_hi, magic_hi);
            uint32_t u2 = and_or(t8, mask_lo, magic_lo), u3 = and_or(t8, mask_hi, magic_hi);
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

// The expert GEMM's K loops are short (6 to 16 blocks) and its grid large: a shallower producer ring keeps the block under
// 128 registers, so three blocks instead of two share a CU.
struct W4MoeTraits : W4Traits {
    static constexpr int PRODUCER_DEPTH = 2;
};

extern "C" __global__ __launch_bounds__(320) void rd_k_gemm_w4a8(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ Xp,
                                                                  float *__restrict__ P, int N, int nKB, int kbPerSplit, int M, int ldP) {
    __shared__ uint4_t lds[2 * RD_LIN_PANEL_BYTES / 16];
    gemm_body<W4Traits, 4, 1, 3>(Wt, nullptr, Xp, P, N, nKB, kbPerSplit, M, ldP, lds);
}
