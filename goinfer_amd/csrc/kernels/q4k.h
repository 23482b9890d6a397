// q4k.h — Q4_K kernels: bit-exact dequantization, re-tiling for coalesced loads, and the dequant-GEMM on f16 MFMA.
//
// Format (goinfer decoder/gguf.go:1508-1537, backend/cuda/actgroup.cu:56-75): a super-block is 256 weights in 144 bytes:
// d f16 @0, dmin f16 @2, 12 bytes of packed 6-bit scales/mins @4, 128 bytes of nibbles @16; w = d*sc_j*q - dmin*m_j.
#pragma once
#include "common.h"
#include "gemm.h"

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

// Re-tile raw row-major super-blocks [N][nSB][144] into [N/32][nSB][4608]: per (row tile, super-block) the 32 headers
// (16 B each), then 4 planes of 64 lanes x 16 B: lane (row r, half h) plane c holds raw code bytes [h*64+c*16, +16) of row r.
// Same bytes, same size; every wave load of the GEMM becomes one contiguous 512 B or 1024 B read.
extern "C" __global__ void rd_k_retile_q4k(const uint8_t *__restrict__ raw, uint8_t *__restrict__ tiled, int N, int nSB) {
    int tile = blockIdx.x, sb = blockIdx.y;
    int t = threadIdx.x; // 0..287: 288 x 16 B = 4608 B
    if (t >= 288) return;
    uint8_t *dst = tiled + ((size_t)tile * nSB + sb) * RD_Q4K_TILE_BYTES;
    const uint4_t *src;
    if (t < 32) {
        src = (const uint4_t *)(raw + ((size_t)(tile * 32 + t) * nSB + sb) * 144);
    } else {
        int u = t - 32, c = u >> 6, lane = u & 63, r = lane & 31, h = lane >> 5;
        src = (const uint4_t *)(raw + ((size_t)(tile * 32 + r) * nSB + sb) * 144 + 16 + h * 64 + c * 16);
    }
    *(uint4_t *)(dst + (size_t)t * 16) = *src;
}

// (a & b) | c in one VALU op. Both constants must sit in VGPRs: a VOP3 instruction on this ISA takes no literal and at
// most one scalar operand, so the compiler otherwise emits v_and + v_or.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t b, uint32_t c) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

struct Q4KTile {
    uint4_t hdr, q[4];
};

__device__ __forceinline__ void q4k_tile_load(Q4KTile &w, const uint8_t *__restrict__ p, int lane) {
    w.hdr = __builtin_nontemporal_load((const uint4_t *)(p + (lane & 31) * 16));
#pragma unroll
    for (int c = 0; c < 4; c++) w.q[c] = __builtin_nontemporal_load((const uint4_t *)(p + 512 + c * 1024 + lane * 16));
}

// acc += panel(32 batch rows x 256 k) . tile(32 weight rows x 256 k)^T, f16 MFMA with f32 accumulation.
// Weights are dequantized in registers: nibble -> f16 via the exponent trick (0x6400|q = 1024+q, 0x5400|(q<<4) = 64+q),
// then one packed fma per pair yields the centred weight (q-8)*dsc rounded once. The per-sub-block constants
// 8*dsc - dmin*m ride a 17th MFMA step against the per-group activation sums.
__device__ __forceinline__ void q4k_tile_mma(float16_t &acc, const Q4KTile &w, const uint4_t *__restrict__ panel, int lane) {
    const int h = lane >> 5;
    const uint32_t mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic_lo = 0x64006400u, magic_hi = 0x54005400u;
    uint32_t y = w.hdr.y, z = w.hdr.z, x = w.hdr.w;
    half2_t dd;
    uint32_t hx = w.hdr.x;
    __builtin_memcpy(&dd, &hx, 4);
    float d = (float)dd.x, dmin = (float)dd.y;
    // Centred form: w = (q-8)*dsc + (8*dsc - dmin*m). The fma constant c = f16(-(1024+8)*dsc) is inexact; its exact
    // remainder delta = c + 1032*dsc is a per-sub-block constant and moves into the offset term, so each weight is
    // rounded exactly once: fma(1024+q, dsc, c) = f16((q-8)*dsc + delta).
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
        const float bias = (jj & 1) ? 72.f : 1032.f; // odd sub-blocks decode as 64+q, even ones as 1024+q
        half_t c = (half_t)(-bias * dscf);
        float delta = (float)c + bias * dscf;
        DSC[jj] = (half2_t){dsc, dsc};
        C0[jj] = (half2_t){c, c};
        off[jj] = (half_t)(8.f * dsc32 - delta - dmin * (float)m); // exact scale here keeps the scale rounding centred
    }
#pragma unroll
    for (int s = 0; s < 16; s++) {
        uint32_t wd = w.q[s >> 2][s & 3];
        const int pp = s >> 3;
        uint32_t t8 = wd >> 8;
        uint32_t u0 = and_or(wd, mask_lo, magic_lo), u1 = and_or(wd, mask_hi, magic_hi);
        uint32_t u2 = and_or(t8, mask_lo, magic_lo), u3 = and_or(t8, mask_hi, magic_hi);
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

// The tile product against MT panels (M-tiles of 32 batch rows): each step's weights are dequantized once and multiplied
// against every M-tile in use. Per M-tile the MFMA sequence is q4k_tile_mma's. mtStride: vectors between the M-tiles' buffers.
template <int MT>
__device__ __forceinline__ void q4k_tile_mma_wide(float16_t (&acc)[MT], const Q4KTile &w, const uint4_t *__restrict__ panel, int mtStride, int nMT,
                                                  int lane) {
    const int h = lane >> 5;
    const uint32_t mask_lo = 0x000F000Fu, mask_hi = 0x00F000F0u, magic_lo = 0x64006400u, magic_hi = 0x54005400u;
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
        const float bias = (jj & 1) ? 72.f : 1032.f;
        half_t c = (half_t)(-bias * dscf);
        float delta = (float)c + bias * dscf;
        DSC[jj] = (half2_t){dsc, dsc};
        C0[jj] = (half2_t){c, c};
        off[jj] = (half_t)(8.f * dsc32 - delta - dmin * (float)m);
    }
    // Every M-tile is multiplied, in use or not (an unused one reads whatever its LDS buffer holds and its sums are never
    // stored): no branch stands between the LDS reads and the MFMAs, so the reads of a step go out together. The loop is bound by
    // those reads (one 1 KB LDS read per MFMA and wave): reading a step further ahead changes nothing.
#pragma unroll
    for (int s = 0; s < 16; s++) {
        uint32_t wd = w.q[s >> 2][s & 3];
        const int pp = s >> 3;
        uint32_t t8 = wd >> 8;
        uint32_t u0 = and_or(wd, mask_lo, magic_lo), u1 = and_or(wd, mask_hi, magic_hi);
        uint32_t u2 = and_or(t8, mask_lo, magic_lo), u3 = and_or(t8, mask_hi, magic_hi);
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
        uint4_t av[MT];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) av[mt] = panel[(size_t)mt * mtStride + s * 64 + lane];
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            half8_t a;
            __builtin_memcpy(&a, &av[mt], 16);
            acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[mt], 0, 0, 0);
        }
    }
    {
        half8_t b = {off[0], off[1], off[2], off[3], (half_t)0, (half_t)0, (half_t)0, (half_t)0};
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
            half8_t a;
            uint4_t av = panel[(size_t)mt * mtStride + 16 * 64 + lane];
            __builtin_memcpy(&a, &av, 16);
            acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[mt], 0, 0, 0);
        }
    }
}

struct Q4KTraits {
    typedef Q4KTile Tile;
    static constexpr int TILE_BYTES = RD_Q4K_TILE_BYTES;
    static constexpr int PANEL_VECS = RD_Q4K_PANEL_BYTES / 16;
    static constexpr int PRODUCER_DEPTH = 2; // 17 KB panels: 68 registers each in the producer wave
    static __device__ __forceinline__ void load(Tile &w, const uint8_t *__restrict__ p, int lane) { q4k_tile_load(w, p, lane); }
    static __device__ __forceinline__ void mma(float16_t &acc, const Tile &w, const uint4_t *__restrict__ panel, int lane) {
        q4k_tile_mma(acc, w, panel, lane);
    }
    template <int MT>
    static __device__ __forceinline__ void mma_wide(float16_t (&acc)[MT], const Tile &w, const uint4_t *__restrict__ panel, int mtStride, int nMT,
                                                    int lane) {
        q4k_tile_mma_wide<MT>(acc, w, panel, mtStride, nMT, lane);
    }
    static __device__ __forceinline__ void finish(float16_t &, const void *, int, int) {}
};

// Grid (ceil(N/128), splits), block 320: four consumer waves (one 32-row tile each) and one panel producer.
extern "C" __global__ __launch_bounds__(320) void rd_k_gemm_q4k(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ Xp,
                                                                 float *__restrict__ P, int N, int nSB, int sbPerSplit, int M, int ldP) {
    __shared__ uint4_t lds[2 * RD_Q4K_PANEL_BYTES / 16];
    gemm_body<Q4KTraits, 4, 1, 3>(Wt, nullptr, Xp, P, N, nSB, sbPerSplit, M, ldP, lds);
}

// Up to 128 batch rows per launch (prefill and verify rows): grid (ceil(N/128), splits), block 512 = four consumer waves and
// one panel producer per M-tile of 32 rows; 136 KB of LDS, one block per CU.
#define RD_GEMM_WIDE_MT 4
extern "C" __global__ __launch_bounds__(512) void rd_k_gemm_q4k_wide(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ Xp, size_t xpStride,
                                                                      float *__restrict__ P, size_t pStride, int N, int nSB, int sbPerSplit, int M,
                                                                      int ldP) {
    __shared__ uint4_t lds[RD_GEMM_WIDE_MT * 2 * RD_Q4K_PANEL_BYTES / 16];
    gemm_body_wide<Q4KTraits, 4, RD_GEMM_WIDE_MT, 3>(Wt, nullptr, Xp, xpStride, P, pStride, N, nSB, sbPerSplit, M, ldP, lds);
}

// 33 to 64 rows: two M-tiles, block 384, 68 KB of LDS (two blocks per CU).
extern "C" __global__ __launch_bounds__(384) void rd_k_gemm_q4k_wide2(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ Xp, size_t xpStride,
                                                                       float *__restrict__ P, size_t pStride, int N, int nSB, int sbPerSplit, int M,
                                                                       int ldP) {
    __shared__ uint4_t lds[2 * 2 * RD_Q4K_PANEL_BYTES / 16];
    gemm_body_wide<Q4KTraits, 4, 2, 3>(Wt, nullptr, Xp, xpStride, P, pStride, N, nSB, sbPerSplit, M, ldP, lds);
}

// Fused gate/up projection + SwiGLU + per-32 quantization (goinfer decoder/cpu_gateup_fused.go:83-148, in one launch):
// W holds [gate rows; up rows] (2*I rows). Block b: waves 0,1 own gate tiles 2b,2b+1, waves 2,3 the matching up tiles, all over
// the full K (no split, so the sums are complete in registers). The up waves hand their sums over through LDS; the gate waves
// compute silu(gate)*up (silu in f64, decoder/rmsnorm.go:204-207), quantize each row's 32 columns (one activation group) and write
// the f16 panels the down projection reads. Each tile's K range is shared by two waves (K-groups) whose partial sums are
// folded in LDS first.
template <int KG, int PF>
__device__ __forceinline__ void q4k_gateup_body(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ Xp, uint8_t *__restrict__ XpOut,
                                                int outKind, int I, int nSB, int M, uint4_t *lds) {
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, wt = wave & 3;
    const int isUp = wt >> 1, t = blockIdx.x * 2 + (wt & 1), nGate = I >> 5;
    const int tile = isUp * nGate + t;
    const bool active = t < nGate;
    float16_t acc;
    const int ltile = active ? tile : nGate - 1;
    gemm_mainloop_pc<Q4KTraits, 4, KG, PF>(acc, Wt + (size_t)ltile * nSB * RD_Q4K_TILE_BYTES, Xp, 0, nSB, lds);
    gemm_fold_groups<4, KG>(acc, (float *)lds);
    // Epilogue on all waves: the four complete tiles (gate t0,t1, up t0,t1) go to LDS as [tile][row m][column c]; then
    // every thread takes elements (tile pair, m, c) with 32 consecutive lanes on one row's 32 columns = one activation group.
    float *xe = (float *)lds + (KG - 1) * 4 * 1024; // 4 tiles x 32 x 32 floats past the fold area
    if (wave < 4) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            xe[(wt * 32 + m) * 32 + (lane & 31)] = acc[r];
        }
    }
    __syncthreads();
    constexpr int NTHR = 4 * KG * 64;
#pragma unroll
    for (int e = tid; e < 2048 && tid < NTHR; e += NTHR) { // consumer waves only; whole waves drop out together
        const int tl = e >> 10, m = (e >> 5) & 31, c = e & 31;
        const int tt = blockIdx.x * 2 + tl;
        float a = __fmul_rn(silu_f64(xe[(tl * 32 + m) * 32 + c]), xe[((2 + tl) * 32 + m) * 32 + c]);
        float gs, xh = quant_g32(a, &gs);
        if (m < M && tt < nGate) {
            int k = tt * 32 + c;
            half_t *base = (half_t *)(XpOut + (size_t)(k >> 8) * RD_Q4K_PANEL_BYTES);
            if (outKind == 0) {
                int t8 = k & 255, j = t8 >> 5;
                base[q4k_panel_index(t8, m)] = (half_t)xh;
                if (c == 0) base[q4k_panel_sum_index(j, m)] = (half_t)gs;
                if (c == 1) base[q4k_panel_sum_index(j, m) + 4] = (half_t)0.f;
            } else {
                half_t *b2 = (half_t *)(XpOut + (size_t)(k >> 7) * RD_LIN_PANEL_BYTES);
                b2[outKind == 1 ? lin_panel_index(k & 127, m) : lin4_panel_index(k & 127, m)] = (half_t)xh;
            }
        }
    }
}

// Grid (I/64), block 640: two K-groups of four consumer waves (gate t0,t1, up t0,t1) plus one producer each.
extern "C" __global__ __launch_bounds__(640) void rd_k_gemm_q4k_gateup(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ Xp,
                                                                        uint8_t *__restrict__ XpOut, int outKind, int I, int nSB, int M) {
    __shared__ uint4_t lds[2 * 2 * RD_Q4K_PANEL_BYTES / 16];
    q4k_gateup_body<2, 3>(Wt, Xp, XpOut, outKind, I, nSB, M, lds);
}
