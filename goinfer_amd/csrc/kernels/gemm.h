// gemm.h — the dequant-GEMM skeleton shared by the Q4_K, int8 and int4-g32 weight kinds.
//
// P[split][32][N] = panels . tiles^T for M <= 32 batch rows. Grid (ceil(N/(32*WPB)), splits), block WPB*64 threads.
// Each wave owns one 32-row weight tile and streams its K-blocks from HBM with two tiles in flight; the block shares the
// activation panel of the current K-block through LDS (double buffered, one barrier per K-block). The reduction order of
// every output element is fixed by (K-block order, MFMA step order) and does not depend on M or on the other rows, so a
// row computed in a batch is bit-identical to the same row computed alone.
#pragma once
#include "common.h"
#include <type_traits>

// acc += panels[kb0,kb1) . (the wave's tile stream at wbase)^T. Every wave of the block must call this (barriers inside).
// Software pipeline: weight tiles are PF K-blocks ahead in registers; the activation panel of K-block it+2 is in flight
// (global -> registers) while it is computed and is published to the LDS buffer vacated one barrier earlier.
// Every load in the loop body is unconditional (indices are clamped to the last K-block, so the tail re-reads it):
// with a fixed number of loads per iteration the compiler can wait for exactly the load it needs (s_waitcnt vmcnt(n))
// and leave the prefetches in flight; conditional loads force it to drain the whole queue.
template <class T, int WPB, int PF = 3>
__device__ __forceinline__ void gemm_mainloop(float16_t &acc, const uint8_t *__restrict__ wbase, const uint8_t *__restrict__ Xp, int kb0, int kb1,
                                              bool active, uint4_t *lds) {
    (void)active; // inactive waves run on a clamped tile (the caller clamps wbase) and simply do not store
    const int tid = threadIdx.x, lane = tid & 63;
    constexpr int PV = T::PANEL_VECS;
    constexpr int NT = WPB * 64;
    constexpr int PER = (PV + NT - 1) / NT;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
    const int nk = kb1 - kb0;
    if (nk <= 0) return;
    const int last = nk - 1;
    const uint8_t *wb = wbase + (size_t)kb0 * T::TILE_BYTES;
    const uint4_t *src = (const uint4_t *)Xp + (size_t)kb0 * PV;
    // vector index of this thread's PER panel slices (the last slice is clamped; its duplicate writes carry the same data)
    int pv[PER];
#pragma unroll
    for (int i = 0; i < PER; i++) pv[i] = min(tid + i * NT, PV - 1);

    typename T::Tile w[PF];
#pragma unroll
    for (int i = 0; i < PF; i++) T::load(w[i], wb + (size_t)min(i, last) * T::TILE_BYTES, lane);
    uint4_t stage[PER];
#pragma unroll
    for (int i = 0; i < PER; i++) lds[pv[i]] = src[pv[i]];
#pragma unroll
    for (int i = 0; i < PER; i++) stage[i] = src[(size_t)min(1, last) * PV + pv[i]];
    __syncthreads();

    auto body = [&](int it, auto uc) {
        constexpr int u = decltype(uc)::value;
        const int cur = it & 1;
        uint4_t *dst = lds + (cur ^ 1) * PV;
#pragma unroll
        for (int i = 0; i < PER; i++) dst[pv[i]] = stage[i]; // panel it+1 (or a harmless copy of the last one)
        const uint4_t *s2 = src + (size_t)min(it + 2, last) * PV;
#pragma unroll
        for (int i = 0; i < PER; i++) stage[i] = s2[pv[i]];
        T::mma(acc, w[u], lds + cur * PV, lane);
        T::load(w[u], wb + (size_t)min(it + PF, last) * T::TILE_BYTES, lane);
        __syncthreads();
    };
    int it = 0;
    for (; it + PF <= nk; it += PF) {
        if constexpr (PF > 0) body(it + 0, std::integral_constant<int, 0>{});
        if constexpr (PF > 1) body(it + 1, std::integral_constant<int, 1>{});
        if constexpr (PF > 2) body(it + 2, std::integral_constant<int, 2>{});
        if constexpr (PF > 3) body(it + 3, std::integral_constant<int, 3>{});
    }
    if constexpr (PF > 1)
        if (it + 0 < nk) body(it + 0, std::integral_constant<int, 0>{});
    if constexpr (PF > 2)
        if (it + 1 < nk) body(it + 1, std::integral_constant<int, 1>{});
    if constexpr (PF > 3)
        if (it + 2 < nk) body(it + 2, std::integral_constant<int, 2>{});
}

// The K-group main loop: a block of TPB*KG waves; wave w owns tile (w % TPB) and K-group (w / TPB). The block's K range
// [kb0,kb1) is cut into KG contiguous runs of `per` K-blocks; each group streams its own run with its own double-buffered
// panel in LDS (lds holds KG*2*PANEL_VECS vectors), all groups share the block barrier. Twice the waves per tile means
// twice the weight bytes in flight per CU — what the HBM latency-bandwidth product asks for — at an unchanged grid.
// A group whose run is shorter than `per` keeps loading (clamped) but skips the arithmetic. acc holds the group's partial
// sum; the caller folds the groups in ascending order (gemm_fold_groups), so the order is fixed and independent of M.
template <class T, int TPB, int KG, int PF = 3>
__device__ __forceinline__ void gemm_mainloop_kg(float16_t &acc, const uint8_t *__restrict__ wbase, const uint8_t *__restrict__ Xp, int kb0, int kb1,
                                                 uint4_t *lds_all) {
    const int tid = threadIdx.x, lane = tid & 63, g = (tid >> 6) / TPB;
    constexpr int PV = T::PANEL_VECS;
    constexpr int NT = TPB * 64; // threads of one group
    constexpr int PER = (PV + NT - 1) / NT;
    const int gtid = tid - g * NT;
    uint4_t *lds = lds_all + g * 2 * PV;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
    const int nkAll = kb1 - kb0;
    if (nkAll <= 0) return;
    const int per = (nkAll + KG - 1) / KG; // block-uniform iteration count
    const int s0 = min(kb0 + g * per, kb1 - 1);
    const int nk = max(0, min(kb1, kb0 + g * per + per) - (kb0 + g * per));
    const int last = max(nk - 1, 0);
    const uint8_t *wb = wbase + (size_t)s0 * T::TILE_BYTES;
    const uint4_t *src = (const uint4_t *)Xp + (size_t)s0 * PV;
    int pv[PER];
#pragma unroll
    for (int i = 0; i < PER; i++) pv[i] = min(gtid + i * NT, PV - 1);

    typename T::Tile w[PF];
#pragma unroll
    for (int i = 0; i < PF; i++) T::load(w[i], wb + (size_t)min(i, last) * T::TILE_BYTES, lane);
    uint4_t stage[PER];
#pragma unroll
    for (int i = 0; i < PER; i++) lds[pv[i]] = src[pv[i]];
#pragma unroll
    for (int i = 0; i < PER; i++) stage[i] = src[(size_t)min(1, last) * PV + pv[i]];
    __syncthreads();

    auto body = [&](int it, auto uc) {
        constexpr int u = decltype(uc)::value;
        const int cur = it & 1;
        uint4_t *dst = lds + (cur ^ 1) * PV;
#ifndef RD_DBG_NO_PANEL
#pragma unroll
        for (int i = 0; i < PER; i++) dst[pv[i]] = stage[i];
        const uint4_t *s2 = src + (size_t)min(it + 2, last) * PV;
#pragma unroll
        for (int i = 0; i < PER; i++) stage[i] = s2[pv[i]];
#endif
        if (it < nk) T::mma(acc, w[u], lds + cur * PV, lane);
        T::load(w[u], wb + (size_t)min(it + PF, last) * T::TILE_BYTES, lane);
#ifndef RD_DBG_NO_BARRIER
        __syncthreads();
#endif
    };
    int it = 0;
    for (; it + PF <= per; it += PF) {
        if constexpr (PF > 0) body(it + 0, std::integral_constant<int, 0>{});
        if constexpr (PF > 1) body(it + 1, std::integral_constant<int, 1>{});
        if constexpr (PF > 2) body(it + 2, std::integral_constant<int, 2>{});
        if constexpr (PF > 3) body(it + 3, std::integral_constant<int, 3>{});
    }
    if constexpr (PF > 1)
        if (it + 0 < per) body(it + 0, std::integral_constant<int, 0>{});
    if constexpr (PF > 2)
        if (it + 1 < per) body(it + 1, std::integral_constant<int, 1>{});
    if constexpr (PF > 3)
        if (it + 2 < per) body(it + 2, std::integral_constant<int, 2>{});
}

// Folds the K-groups' partial sums into group 0's registers in ascending group order through LDS (xch: (KG-1)*TPB*1024
// floats, may alias the panel buffers: the main loop ends on a barrier). Every wave of the block must call it.
template <int TPB, int KG>
__device__ __forceinline__ void gemm_fold_groups(float16_t &acc, float *xch) {
    if constexpr (KG > 1) {
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = wave / TPB, t = wave % TPB;
        if (g > 0) {
#pragma unroll
            for (int r = 0; r < 16; r++) xch[(((g - 1) * TPB + t) * 16 + r) * 64 + lane] = acc[r];
        }
        __syncthreads();
        if (g == 0) {
#pragma unroll
            for (int gg = 1; gg < KG; gg++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[r] += xch[(((gg - 1) * TPB + t) * 16 + r) * 64 + lane];
        }
    }
}

// gemm_body with K-groups: grid (ceil(N/(32*TPB)), splits), block TPB*KG*64 threads.
template <class T, int TPB, int KG, int PF>
__device__ __forceinline__ void gemm_body_kg(const uint8_t *__restrict__ Wt, const void *__restrict__ aux, const uint8_t *__restrict__ Xp,
                                             float *__restrict__ P, int N, int nKB, int kbPerSplit, int M, uint4_t *lds) {
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int tile = blockIdx.x * TPB + wave % TPB, split = blockIdx.y;
    const int kb0 = split * kbPerSplit, kb1 = min(nKB, kb0 + kbPerSplit);
    const bool active = tile * 32 < N;
    float16_t acc;
    const int ltile = active ? tile : (N >> 5) - 1;
    gemm_mainloop_kg<T, TPB, KG, PF>(acc, Wt + (size_t)ltile * nKB * T::TILE_BYTES, Xp, kb0, kb1, lds);
    gemm_fold_groups<TPB, KG>(acc, (float *)lds);
    if (active && kb0 < kb1 && wave < TPB) {
        T::finish(acc, aux, tile, lane);
        float *out = P + (size_t)split * 32 * N + tile * 32 + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; r++) {
            int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            if (m < M) out[(size_t)m * N] = acc[r];
        }
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
#ifndef RD_STREAM_PF
#define RD_STREAM_PF 3
#endif
    const int ltile = active ? tile : (N >> 5) - 1;
    gemm_mainloop<T, WPB, RD_STREAM_PF>(acc, Wt + (size_t)ltile * nKB * T::TILE_BYTES, Xp, kb0, kb1, active, lds);
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

// The resident-panel variant: the block first brings the NP activation panels of its K range into LDS (one barrier), then
// every wave streams its weight tiles with PF tiles in flight and no further synchronisation. It is the right shape when a
// GEMM has too few blocks to hide a per-K-block barrier behind other blocks (the decode projections: a few MB each).
// Same per-element reduction order as the streaming variant within a split.
template <class T, int WPB, int NP, int PF>
__device__ __forceinline__ void gemm_resident_body(const uint8_t *__restrict__ Wt, const void *__restrict__ aux, const uint8_t *__restrict__ Xp,
                                                   float *__restrict__ P, int N, int nKB, int M, uint4_t *lds) {
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int tile = blockIdx.x * WPB + wave, split = blockIdx.y;
    const int kb0 = split * NP, nk = min(NP, nKB - kb0);
    const bool active = tile * 32 < N;
    constexpr int PV = T::PANEL_VECS, NT = WPB * 64;
    const uint8_t *wbase = Wt + ((size_t)tile * nKB + kb0) * T::TILE_BYTES;
    typename T::Tile w[PF];
#pragma unroll
    for (int i = 0; i < PF; i++)
        if (active && i < nk) T::load(w[i], wbase + (size_t)i * T::TILE_BYTES, lane);
    {
        const uint4_t *src = (const uint4_t *)Xp + (size_t)kb0 * PV;
        const int total = nk * PV;
        for (int base = 0; base < total; base += NT * 8) {
            uint4_t r[8];
#pragma unroll
            for (int j = 0; j < 8; j++) {
                int v = base + j * NT + tid;
                if (v < total) r[j] = src[v];
            }
#pragma unroll
            for (int j = 0; j < 8; j++) {
                int v = base + j * NT + tid;
                if (v < total) lds[v] = r[j];
            }
        }
    }
    __syncthreads();
    if (!active) return;
    float16_t acc;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
#pragma unroll
    for (int i = 0; i < NP; i++) {
        if (i < nk) {
            T::mma(acc, w[i % PF], lds + i * PV, lane);
            if (i + PF < nk) T::load(w[i % PF], wbase + (size_t)(i + PF) * T::TILE_BYTES, lane);
        }
    }
    T::finish(acc, aux, tile, lane);
    float *out = P + (size_t)split * 32 * N + tile * 32 + (lane & 31);
#pragma unroll
    for (int r = 0; r < 16; r++) {
        int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (m < M) out[(size_t)m * N] = acc[r];
    }
}
