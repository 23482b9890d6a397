// topk.h — a logits row reduced on the device to its K best entries, for sampled decode with a top-k / min-p / top-p filter
// (goinfer: resident.TopKRow, decoder/resident/forward.go:86-96; the host sampler that consumes it,
// internal/runtime/sampling/sampler_topk.go:10-120; the CUDA counterpart, backend/cuda/topk.cu).
//
// Contract: the first K of the row sorted by (logit DESCENDING, token id ASCENDING) — the order of the host's topKByLogit
// (sampler.go:726-745: ties evict larger ids), with -0 and +0 equal as they are to its '!=' — the entries' own values, and,
// when asked, Z = sum over the whole row of exp((l - max) * invT), the softmax denominator top-p's nucleus cut needs.
//
// One block of 1024 threads per row, the row read from L2 a few times and never copied: an exact radix select on an
// order-preserving 32-bit key in four 8-bit passes (per-wave histograms in LDS, so no two waves contend), then every wave
// gathers, from a contiguous segment of the row, the entries above the K-th key and its share of the first `need` entries
// equal to it (segments ascend with the wave index and lanes with the token id, so "first" is by ascending id), a bitonic
// sort of the at most 1024 survivors in LDS, and one more pass for Z: exp in f32 as the CUDA kernel's, summed in f64 in a
// fixed order (lane-strided per thread, wave butterfly, waves in order).
#pragma once
#include "common.h"

#define RD_TOPK_MAX 1024
#define RD_TOPK_THREADS 1024

// larger float <=> larger key; -0 is +0
__device__ __forceinline__ uint32_t topk_key(float x) {
    if (x == 0.f) x = 0.f;
    const uint32_t u = __float_as_uint(x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ bool topk_before(float av, int ai, float bv, int bi) { return av > bv || (av == bv && ai < bi); }

// Grid (rows), block 1024. logits: [rows][V]; ids_out, vals_out: [rows][k]; z_out (may be NULL): [rows] f64; invTRows (may be
// NULL: every row uses invT): 1/T per row. k <= min(V, 1024).
extern "C" __global__ __launch_bounds__(RD_TOPK_THREADS) void rd_k_topk_rows(const float *__restrict__ logits, int V, int k, float invT,
                                                                             const float *__restrict__ invTRows, int *__restrict__ ids_out,
                                                                             float *__restrict__ vals_out, double *__restrict__ z_out) {
    constexpr int NW = RD_TOPK_THREADS / 64;
    __shared__ int hist[NW][256];
    __shared__ int total[256];
    __shared__ float sval[RD_TOPK_MAX];
    __shared__ int sidx[RD_TOPK_MAX];
    __shared__ int wgt[NW], weq[NW];
    __shared__ double wz[NW];
    __shared__ uint32_t s_prefix;
    __shared__ int s_need, s_greater;
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
    const float *row = logits + (size_t)blockIdx.x * V;

    // ---- the K-th largest key: four 8-bit digits, most significant first ----
    if (t == 0) s_prefix = 0u, s_need = k, s_greater = 0;
    for (int pass = 0; pass < 4; pass++) {
        const int shift = 24 - 8 * pass;
        for (int i = t; i < NW * 256; i += RD_TOPK_THREADS) (&hist[0][0])[i] = 0;
        __syncthreads();
        const uint32_t prefix = s_prefix;
        for (int i = t; i < V; i += RD_TOPK_THREADS) {
            const uint32_t kx = topk_key(row[i]);
            if (pass == 0 || (kx >> (shift + 8)) == prefix) atomicAdd(&hist[wave][(kx >> shift) & 255], 1);
        }
        __syncthreads();
        if (t < 256) {
            int s = 0;
#pragma unroll
            for (int w = 0; w < NW; w++) s += hist[w][t];
            total[t] = s;
        }
        __syncthreads();
        if (t == 0) {
            int need = s_need, cum = 0, b = 255;
            for (; b > 0; b--) {
                if (cum + total[b] >= need) break;
                cum += total[b];
            }
            s_need = need - cum; // how many of digit b's entries are still wanted
            s_greater += cum;
            s_prefix = (prefix << 8) | (uint32_t)b;
        }
        __syncthreads();
    }
    const uint32_t kth = s_prefix;
    const int greater = s_greater, need = s_need; // greater + need == k

    // ---- gather: wave w owns the contiguous segment [w*seg, (w+1)*seg) ----
    const int seg = (V + NW - 1) / NW, lo = wave * seg, hi = min(V, lo + seg);
    int ng = 0, ne = 0;
    for (int i = lo + lane; i < hi; i += 64) {
        const uint32_t kx = topk_key(row[i]);
        ng += kx > kth, ne += kx == kth;
    }
    for (int o = 32; o > 0; o >>= 1) ng += __shfl_xor(ng, o, 64), ne += __shfl_xor(ne, o, 64);
    if (lane == 0) wgt[wave] = ng, weq[wave] = ne;
    __syncthreads();
    int gpos = 0, epos = 0; // where this wave's entries start among the greater ones and among the equal ones
    for (int w = 0; w < wave; w++) gpos += wgt[w], epos += weq[w];
    const unsigned long long below = (1ull << lane) - 1ull;
    for (int base = lo; base < hi; base += 64) {
        const int i = base + lane;
        float x = 0.f;
        bool g = false, e = false;
        if (i < hi) {
            x = row[i];
            const uint32_t kx = topk_key(x);
            g = kx > kth, e = kx == kth;
        }
        const unsigned long long mg = __ballot(g), me = __ballot(e);
        if (g) {
            const int p = gpos + __popcll(mg & below);
            sval[p] = x, sidx[p] = i;
        }
        if (e) {
            const int p = epos + __popcll(me & below);
            if (p < need) sval[greater + p] = x, sidx[greater + p] = i;
        }
        gpos += __popcll(mg), epos += __popcll(me);
    }
    // pad to the sort's power of two with entries that sort last
    int P = 1;
    while (P < k) P <<= 1;
    __syncthreads();
    for (int i = k + t; i < P; i += RD_TOPK_THREADS) sval[i] = -INFINITY, sidx[i] = 0x7fffffff;
    __syncthreads();

    // ---- bitonic sort into (value descending, id ascending) ----
    for (int kk = 2; kk <= P; kk <<= 1) {
        for (int j = kk >> 1; j > 0; j >>= 1) {
            const int i = t, ixj = i ^ j;
            if (i < P && ixj > i) {
                const bool up = (i & kk) == 0;
                const bool ib = topk_before(sval[i], sidx[i], sval[ixj], sidx[ixj]);
                if (up ? !ib : ib) {
                    const float tv = sval[i];
                    sval[i] = sval[ixj], sval[ixj] = tv;
                    const int ti = sidx[i];
                    sidx[i] = sidx[ixj], sidx[ixj] = ti;
                }
            }
            __syncthreads();
        }
    }
    for (int i = t; i < k; i += RD_TOPK_THREADS) ids_out[(size_t)blockIdx.x * k + i] = sidx[i], vals_out[(size_t)blockIdx.x * k + i] = sval[i];

    // ---- Z over the whole row ----
    if (z_out) {
        const float mx = sval[0];
        if (invTRows) invT = invTRows[blockIdx.x];
        double acc = 0.0;
        for (int i = t; i < V; i += RD_TOPK_THREADS) acc += (double)expf(__fmul_rn(__fsub_rn(row[i], mx), invT));
        for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
        if (lane == 0) wz[wave] = acc;
        __syncthreads();
        if (t == 0) {
            double z = 0.0;
            for (int w = 0; w < NW; w++) z += wz[w];
            z_out[blockIdx.x] = z;
        }
    }
}
