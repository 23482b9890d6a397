// gemm.h — the f16-MFMA dequant-GEMM skeleton of the Q5_K and Q6_K weight kinds (kquant.h).
//
// P[split][32][N] = panels . tiles^T for M <= 32 batch rows. Grid (ceil(N/(32*TPB)), splits), block (TPB+1)*KG waves.
// Each consumer wave owns one 32-row weight tile and streams its K-blocks from HBM with PF tiles in flight; producer waves
// keep the activation panel of the next K-block coming through LDS (double buffered, one barrier per K-block). The
// reduction order of every output element is fixed by (K-group, K-block, MFMA step) and does not depend on M or on the
// other rows, so a row computed in a batch is bit-identical to the same row computed alone.
#pragma once
#include "common.h"
#include <type_traits>

// The producer/consumer main loop. Loads return in issue order as far as a wave's wait counter is concerned, so a wave that
// both streams weights and stages activation panels must, when it waits for a panel, also wait for every weight tile it
// asked for earlier: one tile stays in flight and the kernel runs at a third of the HBM rate. Here the roles are split:
// waves 0 .. TPB*KG-1 are consumers (tile w % TPB, K-group w / TPB) whose only global loads are weight tiles, PF deep, and
// waves TPB*KG + g are producers that move group g's panels global -> registers -> LDS one K-block ahead of the consumers
// (T::PRODUCER_DEPTH K-blocks ahead in flight). Block (TPB+1)*KG waves, one barrier per K-block shared by all, LDS KG*2*PANEL_VECS
// vectors. Every wave executes 1 + per barriers. acc is meaningful in consumer waves only.
template <class T, int TPB, int KG, int PF>
__device__ __forceinline__ void gemm_mainloop_pc(float16_t &acc, const uint8_t *__restrict__ wbase, const uint8_t *__restrict__ Xp, int kb0, int kb1,
                                                 uint4_t *lds_all) {
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int PV = T::PANEL_VECS, PVL = PV / 64;
    static_assert(PV % 64 == 0, "panel must be a whole number of 1 KB wave loads");
    const bool producer = wave >= TPB * KG;
    const int g = producer ? wave - TPB * KG : wave / TPB;
    uint4_t *lds = lds_all + g * 2 * PV;
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
    const int nkAll = kb1 - kb0;
    if (nkAll <= 0) return;
    const int per = (nkAll + KG - 1) / KG; // block-uniform iteration count
    const int s0 = min(kb0 + g * per, kb1 - 1);
    const int nk = max(0, min(kb1, kb0 + g * per + per) - (kb0 + g * per));
    const int last = max(nk - 1, 0);
    if (producer) {
        // ring[slot] holds panel it+1 at the top of iteration it (slot = it % PD) and is refilled with panel it+1+PD once
        // written to LDS: PD panels in flight, so the L2 latency is spread over PD K-blocks of consumer work.
        constexpr int PD = T::PRODUCER_DEPTH;
        const uint4_t *src = (const uint4_t *)Xp + (size_t)s0 * PV + lane;
        uint4_t ring[PD][PVL];
        {
            uint4_t first[PVL];
#pragma unroll
            for (int j = 0; j < PVL; j++) first[j] = src[j * 64];
#pragma unroll
            for (int d = 0; d < PD; d++)
#pragma unroll
                for (int j = 0; j < PVL; j++) ring[d][j] = src[(size_t)min(1 + d, last) * PV + j * 64];
#pragma unroll
            for (int j = 0; j < PVL; j++) lds[j * 64 + lane] = first[j];
        }
        __syncthreads();
        auto pbody = [&](int it, auto sc) {
            constexpr int slot = decltype(sc)::value;
            uint4_t *dst = lds + ((it + 1) & 1) * PV + lane;
#pragma unroll
            for (int j = 0; j < PVL; j++) dst[j * 64] = ring[slot][j]; // panel it+1 (a copy of the last one at the tail)
            const uint4_t *s2 = src + (size_t)min(it + 1 + PD, last) * PV;
#pragma unroll
            for (int j = 0; j < PVL; j++) ring[slot][j] = s2[j * 64];
            __syncthreads();
        };
        int it = 0;
        for (; it + PD <= per; it += PD) {
            if constexpr (PD > 0) pbody(it + 0, std::integral_constant<int, 0>{});
            if constexpr (PD > 1) pbody(it + 1, std::integral_constant<int, 1>{});
            if constexpr (PD > 2) pbody(it + 2, std::integral_constant<int, 2>{});
            if constexpr (PD > 3) pbody(it + 3, std::integral_constant<int, 3>{});
        }
        if constexpr (PD > 1)
            if (it + 0 < per) pbody(it + 0, std::integral_constant<int, 0>{});
        if constexpr (PD > 2)
            if (it + 1 < per) pbody(it + 1, std::integral_constant<int, 1>{});
        if constexpr (PD > 3)
            if (it + 2 < per) pbody(it + 2, std::integral_constant<int, 2>{});
        return;
    }
    const uint8_t *wb = wbase + (size_t)s0 * T::TILE_BYTES;
    typename T::Tile w[PF];
#pragma unroll
    for (int i = 0; i < PF; i++) T::load(w[i], wb + (size_t)min(i, last) * T::TILE_BYTES, lane);
    __syncthreads();
    auto body = [&](int it, auto uc) {
        constexpr int u = decltype(uc)::value;
        if (it < nk) T::mma(acc, w[u], lds + (it & 1) * PV, lane);
        T::load(w[u], wb + (size_t)min(it + PF, last) * T::TILE_BYTES, lane);
        __syncthreads();
    };
    int it = 0;
    for (; it + PF <= per; it += PF) {
        if constexpr (PF > 0) body(it + 0, std::integral_constant<int, 0>{});
        if constexpr (PF > 1) body(it + 1, std::integral_constant<int, 1>{});
        if constexpr (PF > 2) body(it + 2, std::integral_constant<int, 2>{});
        if constexpr (PF > 3) body(it + 3, std::integral_constant<int, 3>{});
        if constexpr (PF > 4) body(it + 4, std::integral_constant<int, 4>{});
        if constexpr (PF > 5) body(it + 5, std::integral_constant<int, 5>{});
    }
    if constexpr (PF > 1)
        if (it + 0 < per) body(it + 0, std::integral_constant<int, 0>{});
    if constexpr (PF > 2)
        if (it + 1 < per) body(it + 1, std::integral_constant<int, 1>{});
    if constexpr (PF > 3)
        if (it + 2 < per) body(it + 2, std::integral_constant<int, 2>{});
    if constexpr (PF > 4)
        if (it + 3 < per) body(it + 3, std::integral_constant<int, 3>{});
    if constexpr (PF > 5)
        if (it + 4 < per) body(it + 4, std::integral_constant<int, 4>{});
}

// Folds the K-groups' partial sums into group 0's registers in ascending group order through LDS (xch: (KG-1)*TPB*1024
// floats, may alias the panel buffers: the main loop ends on a barrier). Every wave of the block must call it.
template <int TPB, int KG>
__device__ __forceinline__ void gemm_fold_groups(float16_t &acc, float *xch) {
    if constexpr (KG > 1) {
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = wave / TPB, t = wave % TPB;
        if (g > 0 && g < KG) { // waves past TPB*KG (panel producers) hold no sums
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

// gemm_body on the producer/consumer loop: grid (ceil(N/(32*TPB)), splits), block (TPB+1)*KG*64 threads. P rows are ldP floats
// apart (ldP > N when several weights of different kinds write side by side into one partial-sum buffer); a split past the
// end of K stores zeros, so that every weight of such a group can be launched with the group's split count.
template <class T, int TPB, int KG, int PF>
__device__ __forceinline__ void gemm_body(const uint8_t *__restrict__ Wt, const void *__restrict__ aux, const uint8_t *__restrict__ Xp,
                                             float *__restrict__ P, int N, int nKB, int kbPerSplit, int M, int ldP, uint4_t *lds) {
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int tile = blockIdx.x * TPB + wave % TPB, split = blockIdx.y;
    const int kb0 = split * kbPerSplit, kb1 = min(nKB, kb0 + kbPerSplit);
    const bool active = tile * 32 < N;
    float16_t acc;
    const int ltile = active ? tile : (N >> 5) - 1;
    gemm_mainloop_pc<T, TPB, KG, PF>(acc, Wt + (size_t)ltile * nKB * T::TILE_BYTES, Xp, kb0, kb1, lds);
    gemm_fold_groups<TPB, KG>(acc, (float *)lds);
    if (active && wave < TPB) {
        T::finish(acc, aux, tile, lane);
        float *out = P + (size_t)split * 32 * ldP + tile * 32 + (lane & 31);
#pragma unroll
        for (int r = 0; r < 16; r++) {
            int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            if (m < M) out[(size_t)m * ldP] = acc[r];
        }
    }
}
