// moe.h — expert-major MoE FFN (goinfer decoder/mlp.go:630-726 moeMLPBatchWith; CUDA analogue backend/cuda/moe_rows.cu).
// A decode batch has at most 32 tokens, so one 32-row MFMA tile covers every token: each expert's GEMM runs over all
// token rows at once and stores only the rows routed to it — the ragged token-to-expert grouping costs no gather and
// every expert's weights are streamed exactly once per step. rankOf[token][expert] (from rd_k_moe_route) is the map.
#pragma once
#include "act.h"
#include "lin.h"

// out[(token*k + rank)][N] = panels . W_e^T for the experts that have at least one token. Grid (ceil(N/128), nE), block 320 (four consumer waves and a panel producer).
// xpStride: bytes between the experts' panel sets (0 = all experts read the same panels: the gate/up projections).
// activeBits (may be NULL): the bitmap of experts with a token. Row y of the grid then works on the y-th expert whose bit is set,
// and the rows past the last one exit: the blocks with work are the first in dispatch order, which spreads them evenly over
// the XCDs and CUs (blocks are handed out round-robin; idle ones scattered among them skew that). Without the bitmap row y is
// expert y, and exits when no token chose it.
// The expert grid row `row` works on, or -1 (uniform over the block; every thread must call it).
__device__ __forceinline__ int moe_block_expert(const unsigned *__restrict__ activeBits, const signed char *__restrict__ rankOf, int nE, int T, int row) {
    int e = row;
    if (activeBits) {
        int y = row;
        for (int w = 0; w < (nE + 31) >> 5; w++) {
            unsigned b = activeBits[w];
            const int c = __popc(b);
            if (y < c) {
                for (int i = 0; i < y; i++) b &= b - 1; // drop the y lowest set bits
                return w * 32 + __ffs((int)b) - 1;
            }
            y -= c;
        }
        return -1;
    }
    int mine = ((int)threadIdx.x < T && rankOf[(size_t)threadIdx.x * nE + e] >= 0) ? 1 : 0;
    return __syncthreads_or(mine) ? e : -1;
}

template <int TPB, int PF>
__device__ __forceinline__ void moe_gemm_body(const uint8_t *__restrict__ Wt, size_t wStride, const uint8_t *__restrict__ Xp, size_t xpStride,
                                              float *__restrict__ out, int N, int nKB, int T, int k, const signed char *__restrict__ rankOf, int nE,
                                              const unsigned *__restrict__ activeBits, uint4_t *lds) {
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    // perExpertPanels: every expert reads panels of its own, so all blocks of an expert are placed on one XCD (blocks go to the
    // eight XCDs round-robin in linear order) and its panels are pulled into one L2 instead of eight.
    int bx = blockIdx.x, row = blockIdx.y;
    if (xpStride != 0 && (gridDim.y & 7) == 0) {
        const int gx = gridDim.x, L = row * gx + bx, j = L >> 3;
        row = (j / gx) * 8 + (L & 7), bx = j % gx;
    }
    const int e = moe_block_expert(activeBits, rankOf, nE, T, row);
    if (e < 0) return;
    const int tile = bx * TPB + (wave % TPB);
    const bool active = tile * 32 < N;
    float16_t acc;
    const int ltile = active ? tile : (N >> 5) - 1;
    gemm_mainloop_pc<W4MoeTraits, TPB, 1, PF>(acc, Wt + (size_t)e * wStride + (size_t)ltile * nKB * W4Traits::TILE_BYTES, Xp + (size_t)e * xpStride, 0,
                                              nKB, lds);
    if (!active || wave >= TPB) return;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (m < T) {
            int rank = rankOf[(size_t)m * nE + e];
            if (rank >= 0) out[((size_t)m * k + rank) * N + tile * 32 + (lane & 31)] = acc[r];
        }
    }
}

extern "C" __global__ __launch_bounds__(320) __attribute__((amdgpu_waves_per_eu(7, 7))) void rd_k_gemm_w4a8_moe(const uint8_t *__restrict__ Wt, size_t wStride, const uint8_t *__restrict__ Xp,
                                                                      size_t xpStride, float *__restrict__ out, int N, int nKB, int T, int k,
                                                                      const signed char *__restrict__ rankOf, int nE,
                                                                      const unsigned *__restrict__ activeBits) {
    __shared__ uint4_t lds[2 * RD_LIN_PANEL_BYTES / 16];
    moe_gemm_body<4, 3>(Wt, wStride, Xp, xpStride, out, N, nKB, T, k, rankOf, nE, activeBits, lds);
}
// The experts' gate|up projection with SwiGLU and the per-32 quantization in its epilogue (the expert twin of rd_k_gemm_q4k_gateup;
// same values as rd_k_gemm_w4a8_moe followed by rd_k_moe_swiglu_quant, bit for bit). Wt per expert: [gate rows; up rows] (2*I rows).
// Grid (I/64, nE), block 320: waves 0,1 own gate tiles 2x, 2x+1 of the block's expert, waves 2,3 the matching up tiles, over all
// of K; the sums meet in LDS, and for every token routed to the expert one wave computes silu(gate)*up for the block's 64
// columns (two activation groups), quantizes them and writes them into the expert's down-projection panels XpE. I % 64 == 0.
extern "C" __global__ __launch_bounds__(320) void rd_k_gemm_w4a8_moe_gateup(const uint8_t *__restrict__ Wt, size_t wStride,
                                                                             const uint8_t *__restrict__ Xp, uint8_t *__restrict__ XpE,
                                                                             size_t xpeStride, int I, int nKB, int T,
                                                                             const signed char *__restrict__ rankOf, int nE,
                                                                             const unsigned *__restrict__ activeBits) {
    __shared__ uint4_t lds[2 * RD_LIN_PANEL_BYTES / 16];
    static_assert(2 * RD_LIN_PANEL_BYTES >= 4 * 32 * 32 * 4, "the four finished tiles are exchanged through the panel buffers");
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, wt = wave & 3;
    const int e = moe_block_expert(activeBits, rankOf, nE, T, blockIdx.y);
    if (e < 0) return;
    const int nGate = I >> 5, tile = (wt >> 1) * nGate + blockIdx.x * 2 + (wt & 1);
    float16_t acc;
    gemm_mainloop_pc<W4MoeTraits, 4, 1, 3>(acc, Wt + (size_t)e * wStride + (size_t)tile * nKB * W4Traits::TILE_BYTES, Xp, 0, nKB, lds);
    __syncthreads(); // every wave is done with the panels
    float *xe = (float *)lds; // [tile wt][row m][column c]
    if (wave < 4) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            xe[(wt * 32 + m) * 32 + (lane & 31)] = acc[r];
        }
    }
    __syncthreads();
    if (wave >= 4) return;
    unsigned long long routed = __ballot(lane < T && rankOf[(size_t)lane * nE + e] >= 0);
    const int tl = lane >> 5, c = lane & 31;
    for (int ord = 0; routed; ord++) {
        const int m = __ffsll((long long)routed) - 1;
        routed &= routed - 1;
        if ((ord & 3) != wave) continue; // the routed rows go round the four waves
        const float a = __fmul_rn(silu_f64(xe[(tl * 32 + m) * 32 + c]), xe[((2 + tl) * 32 + m) * 32 + c]);
        float gs, xh = quant_g32(a, &gs); // a half-wave holds the 32 columns of one tile = one activation group
        panel_store(XpE + (size_t)e * xpeStride, RD_PANEL_LIN4, m, (blockIdx.x * 2 + tl) * 32 + c, xh, gs);
    }
}

// gate/up rows [(token,rank)][2I] -> silu(gate)*up -> per-32 quantization -> the down-projection panels of that row's expert.
// Grid (ceil(I/256), T*k).
extern "C" __global__ __launch_bounds__(256) void rd_k_moe_swiglu_quant(const float *__restrict__ gu, const int *__restrict__ idx, int I, int k,
                                                                        uint8_t *__restrict__ XpE, size_t xpStride) {
    int row = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x, t = row / k, e = idx[row];
    float a = 0.f;
    if (n < I) {
        float g = gu[(size_t)row * 2 * I + n], u = gu[(size_t)row * 2 * I + I + n];
        a = __fmul_rn(silu_f64(g), u);
    }
    float gs, xh = quant_g32(a, &gs);
    if (n < I) panel_store(XpE + (size_t)e * xpStride, RD_PANEL_LIN4, t, n, xh, gs);
}

// out[t][:] = sum over ranks, in rank order, of wgt[t][rank] * down[(t,rank)][:]  (decoder/mlp.go:100-103, addScaled: mul then add).
extern "C" __global__ void rd_k_moe_fold(const float *__restrict__ dn, const float *__restrict__ wgt, float *__restrict__ out, int H, int k) {
    int t = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x;
    if (n >= H) return;
    float acc = 0.f;
    for (int r = 0; r < k; r++) acc = __fadd_rn(acc, mul_rounded(wgt[t * k + r], dn[((size_t)t * k + r) * H + n]));
    out[(size_t)t * H + n] = acc;
}
