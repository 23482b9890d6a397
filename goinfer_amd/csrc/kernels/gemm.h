// gemm.h — the dequant-GEMM skeleton shared by the Q4_K, int8 and int4-g32 weight kinds.
//
// P[split][32][N] = panels . tiles^T for M <= 32 batch rows. Grid (ceil(N/(32*WPB)), splits), block WPB*64 threads.
// Each wave owns one 32-row weight tile and streams its K-blocks from HBM with two tiles in flight; the block shares the
// activation panel of the current K-block through LDS (double buffered, one barrier per K-block). The reduction order of
// every output element is fixed by (K-block order, MFMA step order) and does not depend on M or on the other rows, so a
// row computed in a batch is bit-identical to the same row computed alone.
#pragma once
#include "common.h"

// acc += panels[kb0,kb1) . (the wave's tile stream at wbase)^T. Every wave of the block must call this (barriers inside).
template <class T, int WPB>
__device__ __forceinline__ void gemm_mainloop(float16_t &acc, const uint8_t *__restrict__ wbase, const uint8_t *__restrict__ Xp, int kb0, int kb1,
                                              bool active, uint4_t *lds) {
    const int tid = threadIdx.x, lane = tid & 63;
    constexpr int PV = T::PANEL_VECS;
    constexpr int NT = WPB * 64;
    constexpr int PER = (PV + NT - 1) / NT;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
    if (kb0 >= kb1) return;

    typename T::Tile w0, w1;
    if (active) {
        T::load(w0, wbase + (size_t)kb0 * T::TILE_BYTES, lane);
        if (kb0 + 1 < kb1) T::load(w1, wbase + (size_t)(kb0 + 1) * T::TILE_BYTES, lane);
    }
    {
        const uint4_t *src = (const uint4_t *)Xp + (size_t)kb0 * PV;
#pragma unroll
        for (int i = 0; i < PER; i++) {
            int v = tid + i * NT;
            if (v < PV) lds[v] = src[v];
        }
    }
    __syncthreads();
    for (int kb = kb0; kb < kb1; kb++) {
        const int cur = (kb - kb0) & 1;
        uint4_t stage[PER];
        const bool more = kb + 1 < kb1;
        if (more) {
            const uint4_t *src = (const uint4_t *)Xp + (size_t)(kb + 1) * PV;
#pragma unroll
            for (int i = 0; i < PER; i++) {
                int v = tid + i * NT;
                if (v < PV) stage[i] = src[v];
            }
        }
        if (active) {
            T::mma(acc, w0, lds + cur * PV, lane);
            w0 = w1;
            if (kb + 2 < kb1) T::load(w1, wbase + (size_t)(kb + 2) * T::TILE_BYTES, lane);
        }
        if (more) {
            uint4_t *dst = lds + (cur ^ 1) * PV;
#pragma unroll
            for (int i = 0; i < PER; i++) {
                int v = tid + i * NT;
                if (v < PV) dst[v] = stage[i];
            }
        }
        __syncthreads();
    }
}

template <class T, int WPB>
__device__ __forceinline__ void gemm_body(const uint8_t *__restrict__ Wt, const void *__restrict__ aux, const uint8_t *__restrict__ Xp,
                                          float *__restrict__ P, int N, int nKB, int kbPerSplit, int M, uint4_t *lds) {
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int tile = blockIdx.x * WPB + wave, split = blockIdx.y;
    const int kb0 = split * kbPerSplit, kb1 = min(nKB, kb0 + kbPerSplit);
    const bool active = tile * 32 < N;
    float16_t acc;
    gemm_mainloop<T, WPB>(acc, Wt + (size_t)tile * nKB * T::TILE_BYTES, Xp, kb0, kb1, active, lds);
    if (active && kb0 < kb1) {
        T::finish(acc, aux, tile, lane);
        float *out = P + (size_t)split * 32 * N + tile * 32 + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; r++) {
            int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            if (m < M) out[(size_t)m * N] = acc[r];
        }
    }
}
