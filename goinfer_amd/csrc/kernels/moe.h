// moe.h — expert-major MoE FFN (goinfer decoder/mlp.go:630-726 moeMLPBatchWith; CUDA analogue backend/cuda/moe_rows.cu).
// A decode batch has at most 32 tokens, so one 32-row MFMA tile covers every token: each expert's GEMM runs over all
// token rows at once and stores only the rows routed to it — the ragged token-to-expert grouping costs no gather and
// every expert's weights are streamed exactly once per step. rankOf[token][expert] (from rd_k_moe_route) is the map.
#pragma once
#include "act.h"
#include "gemm8.h"

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

// Per expert the weights are W4A8 tiles of the int8-MFMA kernels (gemm8.h: 4608 B per 32 rows x 256 k), the activations A8 blocks.
// Block: TPB tiles x KW waves, every wave on its own K range, partial sums folded through LDS in wave order (as gemm8_body).
template <int KW, int TPB>
__device__ __forceinline__ void moe_gemm8_body(const uint8_t *__restrict__ Wt, size_t wStride, const uint8_t *__restrict__ A8, size_t a8Stride,
                                               float *__restrict__ out, int N, int nKB, int T, int k, const signed char *__restrict__ rankOf, int nE,
                                               const unsigned *__restrict__ activeBits, float *lds) {
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    // a8Stride != 0: every expert reads activations of its own, so all blocks of an expert are placed on one XCD (blocks go to the
    // eight XCDs round-robin in linear order) and its activation blocks are pulled into one L2 instead of eight.
    int bx = blockIdx.x, row = blockIdx.y;
    if (a8Stride != 0 && (gridDim.y & 7) == 0) {
        const int gx = gridDim.x, L = row * gx + bx, j = L >> 3;
        row = (j / gx) * 8 + (L & 7), bx = j % gx;
    }
    const int e = moe_block_expert(activeBits, rankOf, nE, T, row);
    if (e < 0) return;
    const int tile = bx * TPB + wave / KW, kw = wave % KW;
    const bool active = tile * 32 < N;
    const int per = (nKB + KW - 1) / KW, s0 = kw * per, nk = max(0, min(nKB, s0 + per) - s0);
    float16_t acc;
    gemm8_wave_loop<W4A8Traits8>(acc, Wt + (size_t)e * wStride + ((size_t)(active ? tile : 0) * nKB + s0) * W4A8Traits8::TILE_BYTES,
                                 A8 + (size_t)e * a8Stride + (size_t)s0 * RD_A8_BLOCK_BYTES, active ? nk : 0, nullptr, tile, lane);
    gemm8_fold_waves<KW, TPB>(acc, lds);
    if (!active || kw != 0) return;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (m < T) {
            const int rank = rankOf[(size_t)m * nE + e];
            if (rank >= 0) out[((size_t)m * k + rank) * N + tile * 32 + (lane & 31)] = acc[r];
        }
    }
}

// out[(token*k + rank)][N] = A8 . W_e^T for the experts that have at least one token. Grid (ceil(N/64), nE), block 256 (two tiles x two waves).
// a8Stride: bytes between the experts' activation sets (0 = all experts read the same activations: the gate/up projections).
extern "C" __global__ __launch_bounds__(256) void rd_k_gemm8_w4a8_moe(const uint8_t *__restrict__ Wt, size_t wStride, const uint8_t *__restrict__ A8,
                                                                       size_t a8Stride, float *__restrict__ out, int N, int nKB, int T, int k,
                                                                       const signed char *__restrict__ rankOf, int nE,
                                                                       const unsigned *__restrict__ activeBits) {
    __shared__ float lds[2 * 1024];
    moe_gemm8_body<2, 2>(Wt, wStride, A8, a8Stride, out, N, nKB, T, k, rankOf, nE, activeBits, lds);
}

// The experts' gate|up projection with SwiGLU and the per-32 quantization in its epilogue (the expert twin of rd_k_gemm8_q4k_gateup;
// same values as rd_k_gemm8_w4a8_moe followed by rd_k_moe_swiglu_quant, bit for bit: both cut K over two waves). Wt per expert:
// [gate rows; up rows] (2*I rows). Grid (I/32, nE), block 256: waves 0,1 own gate tile x of the block's expert, waves 2,3 the
// matching up tile; the finished tiles meet in LDS in accumulator order, every wave takes four accumulator registers, and the
// rows routed to the expert are quantized (a half-wave holds the 32 columns of one row = one activation group) and written into
// the expert's down-projection activations A8E.
extern "C" __global__ __launch_bounds__(256) void rd_k_gemm8_w4a8_moe_gateup(const uint8_t *__restrict__ Wt, size_t wStride,
                                                                              const uint8_t *__restrict__ A8, uint8_t *__restrict__ A8E,
                                                                              size_t a8eStride, int I, int nKB, int T,
                                                                              const signed char *__restrict__ rankOf, int nE,
                                                                              const unsigned *__restrict__ activeBits) {
    __shared__ float lds[2 * 1024];
    constexpr int KW = 2;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int e = moe_block_expert(activeBits, rankOf, nE, T, blockIdx.y);
    if (e < 0) return;
    const int half = wave / KW, kw = wave % KW, t = blockIdx.x, nGate = I >> 5, tile = half * nGate + t;
    const int per = (nKB + KW - 1) / KW, s0 = kw * per, nk = max(0, min(nKB, s0 + per) - s0);
    float16_t acc;
    gemm8_wave_loop<W4A8Traits8>(acc, Wt + (size_t)e * wStride + ((size_t)tile * nKB + s0) * W4A8Traits8::TILE_BYTES, A8 + (size_t)s0 * RD_A8_BLOCK_BYTES, nk,
                                 nullptr, tile, lane);
    gemm8_fold_waves<KW, 2>(acc, lds);
    __syncthreads();
    if (kw == 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) lds[(half * 16 + r) * 64 + lane] = acc[r];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int r = wave * 4 + j, m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        const bool routed = m < T && rankOf[(size_t)m * nE + e] >= 0;
        if (__ballot(routed) == 0) continue; // no row of this register is routed here: skip the f64 silu
        const float a = __fmul_rn(silu_f64(lds[r * 64 + lane]), lds[(16 + r) * 64 + lane]);
        const Quant1 q = quant_one(a);
        if (routed) panel_store(A8E + (size_t)e * a8eStride, RD_PANEL_A8, m, t * 32 + (lane & 31), q);
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
    const Quant1 q = quant_one(a);
    if (n < I) panel_store(XpE + (size_t)e * xpStride, RD_PANEL_A8, t, n, q);
}

// out[t][:] = sum over ranks, in rank order, of wgt[t][rank] * down[(t,rank)][:]  (decoder/mlp.go:100-103, addScaled: mul then add).
extern "C" __global__ void rd_k_moe_fold(const float *__restrict__ dn, const float *__restrict__ wgt, float *__restrict__ out, int H, int k) {
    int t = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x;
    if (n >= H) return;
    float acc = 0.f;
    for (int r = 0; r < k; r++) acc = __fadd_rn(acc, mul_rounded(wgt[t * k + r], dn[((size_t)t * k + r) * H + n]));
    out[(size_t)t * H + n] = acc;
}
