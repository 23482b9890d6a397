// topk.h — a logits row reduced on the device to its K best entries, for sampled decode with a top-k / min-p / top-p filter
// (goinfer: resident.TopKRow, decoder/resident/forward.go:86-96; the host sampler that consumes it,
// internal/runtime/sampling/sampler_topk.go:10-120; the CUDA counterpart, backend/cuda/topk.cu).
//
// Contract: the first K of the row sorted by (logit DESCENDING, token id ASCENDING) — the order of the host's topKByLogit
// (sampler.go:726-745: ties evict larger ids), with -0 and +0 equal as they are to its '!=' — the entries' own values, and,
// when asked, Z = sum over the whole row of exp((l - max) * invT), the softmax denominator top-p's nucleus cut needs.
//
// Two routes to the same answer. The exact route, below: one block of 1024 threads per row, the row read from L2 a few times and never copied: an exact radix select on an
// order-preserving 32-bit key in four 8-bit passes (per-wave histograms in LDS, so no two waves contend), then every wave
// gathers, from a contiguous segment of the row, the entries above the K-th key and its share of the first `need` entries
// equal to it (segments ascend with the wave index and lanes with the token id, so "first" is by ascending id), a bitonic
// sort of the at most 1024 survivors in LDS, and one more pass for Z: exp in f32 as the CUDA kernel's, summed in f64 in a
// fixed order (lane-strided per thread, wave butterfly, waves in order).
//
// The fast route, for wide rows (rd_k_topk_hist, rd_k_topk_pick, rd_k_topk_finish): the row is spread over the chip in chunks of
// 16384. A first launch histograms the top 11 key bits of every chunk and finds its maximum; a
// second adds the chunks' histograms up, and compacts every entry from the bin that holds the K-th largest upward (a few hundred to a few thousand entries for
// logits) into a candidate list and sums its chunk's share of Z; the last sorts the candidates in LDS and takes the first K.
// That is exact whenever the candidates fit the list, because every entry at or above the threshold bin was collected and at
// least K were; a row whose threshold bin is too crowded (flat or heavily tied rows) takes the exact route inside the last
// launch. The order candidates arrive in does not matter: the sort's key (value, id) is unique.
#pragma once
#include "common.h"

#define RD_TOPK_MAX 1024
#define RD_TOPK_THREADS 1024
#define RD_TOPK_CAP 4096   // candidate list of the fast route, per row
#define RD_TOPK_BINS 2048  // its histogram: the top 11 key bits
#define RD_TOPK_CHUNK 16384 // row entries per block of its two grid launches

// larger float <=> larger key; -0 is +0
__device__ __forceinline__ uint32_t topk_key(float x) {
    if (x == 0.f) x = 0.f;
    const uint32_t u = __float_as_uint(x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float topk_unkey(uint32_t k) { return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k); }
__device__ __forceinline__ bool topk_before(float av, int ai, float bv, int bi) { return av > bv || (av == bv && ai < bi); }

// LDS of the one-block stages (49 KB)
struct TopkShared {
    int hist[RD_TOPK_THREADS / 64][256];
    int total[256];
    float sval[RD_TOPK_CAP];
    int sidx[RD_TOPK_CAP];
    int wgt[RD_TOPK_THREADS / 64], weq[RD_TOPK_THREADS / 64];
    double wz[RD_TOPK_THREADS / 64];
    uint32_t prefix;
    int need, greater;
};

// The exact route's selection: leaves the row's k best entries, unordered, in sh.sval/sidx[0..k). Every thread of the block calls it.
__device__ __forceinline__ void topk_select_exact(const float *__restrict__ row, int V, int k, TopkShared &sh) {
    constexpr int NW = RD_TOPK_THREADS / 64;
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
    // the K-th largest key: four 8-bit digits, most significant first
    __syncthreads();
    if (t == 0) sh.prefix = 0u, sh.need = k, sh.greater = 0;
    for (int pass = 0; pass < 4; pass++) {
        const int shift = 24 - 8 * pass;
        for (int i = t; i < NW * 256; i += RD_TOPK_THREADS) (&sh.hist[0][0])[i] = 0;
        __syncthreads();
        const uint32_t prefix = sh.prefix;
        for (int i = t; i < V; i += RD_TOPK_THREADS) {
            const uint32_t kx = topk_key(row[i]);
            if (pass == 0 || (kx >> (shift + 8)) == prefix) atomicAdd(&sh.hist[wave][(kx >> shift) & 255], 1);
        }
        __syncthreads();
        if (t < 256) {
            int s = 0;
#pragma unroll
            for (int w = 0; w < NW; w++) s += sh.hist[w][t];
            sh.total[t] = s;
        }
        __syncthreads();
        if (t == 0) {
            int need = sh.need, cum = 0, b = 255;
            for (; b > 0; b--) {
                if (cum + sh.total[b] >= need) break;
                cum += sh.total[b];
            }
            sh.need = need - cum; // how many of digit b's entries are still wanted
            sh.greater += cum;
            sh.prefix = (prefix << 8) | (uint32_t)b;
        }
        __syncthreads();
    }
    const uint32_t kth = sh.prefix;
    const int greater = sh.greater, need = sh.need; // greater + need == k
    // gather: wave w owns the contiguous segment [w*seg, (w+1)*seg)
    const int seg = (V + NW - 1) / NW, lo = min(V, wave * seg), hi = min(V, lo + seg);
    int ng = 0, ne = 0;
    for (int i = lo + lane; i < hi; i += 64) {
        const uint32_t kx = topk_key(row[i]);
        ng += kx > kth, ne += kx == kth;
    }
    for (int o = 32; o > 0; o >>= 1) ng += __shfl_xor(ng, o, 64), ne += __shfl_xor(ne, o, 64);
    if (lane == 0) sh.wgt[wave] = ng, sh.weq[wave] = ne;
    __syncthreads();
    int gpos = 0, epos = 0; // where this wave's entries start among the greater ones and among the equal ones
    for (int w = 0; w < wave; w++) gpos += sh.wgt[w], epos += sh.weq[w];
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
            sh.sval[p] = x, sh.sidx[p] = i;
        }
        if (e) {
            const int p = epos + __popcll(me & below);
            if (p < need) sh.sval[greater + p] = x, sh.sidx[greater + p] = i;
        }
        gpos += __popcll(mg), epos += __popcll(me);
    }
    __syncthreads();
}

// Sorts sh.sval/sidx[0..n) into (value descending, id ascending) order; n <= RD_TOPK_CAP. Every thread of the block calls it.
__device__ __forceinline__ void topk_sort(TopkShared &sh, int n) {
    const int t = threadIdx.x;
    int P = 1;
    while (P < n) P <<= 1;
    for (int i = n + t; i < P; i += RD_TOPK_THREADS) sh.sval[i] = -INFINITY, sh.sidx[i] = 0x7fffffff; // entries that sort last
    __syncthreads();
    for (int kk = 2; kk <= P; kk <<= 1) {
        for (int j = kk >> 1; j > 0; j >>= 1) {
            for (int i = t; i < P; i += RD_TOPK_THREADS) {
                const int ixj = i ^ j;
                if (ixj > i) {
                    const bool up = (i & kk) == 0;
                    const bool ib = topk_before(sh.sval[i], sh.sidx[i], sh.sval[ixj], sh.sidx[ixj]);
                    if (up ? !ib : ib) {
                        const float tv = sh.sval[i];
                        sh.sval[i] = sh.sval[ixj], sh.sval[ixj] = tv;
                        const int ti = sh.sidx[i];
                        sh.sidx[i] = sh.sidx[ixj], sh.sidx[ixj] = ti;
                    }
                }
            }
            __syncthreads();
        }
    }
}

// One term of Z (backend/cuda/topk.cu:415-418: the product made explicit, exp in f32)
__device__ __forceinline__ double topk_z_term(float x, float mx, float invT) { return (double)expf(__fmul_rn(__fsub_rn(x, mx), invT)); }

// The exact route in one launch. Grid (rows), block 1024. logits: [rows][V]; ids_out, vals_out: [rows][k]; z_out (may be NULL):
// [rows] f64; invTRows (may be NULL: every row uses invT): 1/T per row. k <= min(V, 1024).
extern "C" __global__ __launch_bounds__(RD_TOPK_THREADS) void rd_k_topk_rows(const float *__restrict__ logits, int V, int k, float invT,
                                                                             const float *__restrict__ invTRows, int *__restrict__ ids_out,
                                                                             float *__restrict__ vals_out, double *__restrict__ z_out) {
    __shared__ TopkShared sh;
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63;
    const float *row = logits + (size_t)blockIdx.x * V;
    topk_select_exact(row, V, k, sh);
    topk_sort(sh, k);
    for (int i = t; i < k; i += RD_TOPK_THREADS) ids_out[(size_t)blockIdx.x * k + i] = sh.sidx[i], vals_out[(size_t)blockIdx.x * k + i] = sh.sval[i];
    if (z_out) { // lane-strided per thread, wave butterfly, waves in order
        const float mx = sh.sval[0];
        if (invTRows) invT = invTRows[blockIdx.x];
        double acc = 0.0;
        for (int i = t; i < V; i += RD_TOPK_THREADS) acc += topk_z_term(row[i], mx, invT);
        for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
        if (lane == 0) sh.wz[wave] = acc;
        __syncthreads();
        if (t == 0) {
            double z = 0.0;
            for (int w = 0; w < RD_TOPK_THREADS / 64; w++) z += sh.wz[w];
            z_out[blockIdx.x] = z;
        }
    }
}

// ---- the fast route ----
// Per-row scratch between its launches: hpart [rows][chunks][RD_TOPK_BINS] and mpart [rows][chunks] (each chunk's histogram and
// largest key, written whole by the first launch); ccount [rows], zero on entry and zero again when the last launch ends;
// cand_v, cand_i [rows][RD_TOPK_CAP]; zpart [rows][chunks] f64.

// Grid (chunks, rows), block 1024: the chunk's histogram of the top 11 key bits and its largest key.
extern "C" __global__ __launch_bounds__(1024) void rd_k_topk_hist(const float *__restrict__ logits, int V, int *__restrict__ hpart,
                                                                  uint32_t *__restrict__ mpart) {
    __shared__ int hist[RD_TOPK_BINS];
    __shared__ uint32_t wmax[16];
    const int t = threadIdx.x, m = blockIdx.y;
    const float *row = logits + (size_t)m * V;
    for (int i = t; i < RD_TOPK_BINS; i += 1024) hist[i] = 0;
    __syncthreads();
    uint32_t mk = 0u;
    const int base = blockIdx.x * RD_TOPK_CHUNK;
#pragma unroll 4
    for (int j = 0; j < RD_TOPK_CHUNK / 1024; j++) {
        const int i = base + j * 1024 + t;
        if (i < V) {
            const uint32_t kx = topk_key(row[i]);
            mk = max(mk, kx);
            atomicAdd(&hist[kx >> 21], 1);
        }
    }
    for (int o = 32; o > 0; o >>= 1) mk = max(mk, (uint32_t)__shfl_xor((int)mk, o, 64));
    if ((t & 63) == 0) wmax[t >> 6] = mk;
    __syncthreads();
    int *dst = hpart + ((size_t)m * gridDim.x + blockIdx.x) * RD_TOPK_BINS;
    for (int i = t; i < RD_TOPK_BINS; i += 1024) dst[i] = hist[i];
    if (t == 0) {
        for (int w = 1; w < 16; w++) mk = max(mk, wmax[w]);
        mpart[(size_t)m * gridDim.x + blockIdx.x] = mk;
    }
}

// Grid (chunks, rows), block 1024: the row's histogram from its chunks', the bin that holds the K-th largest, then every entry
// of this block's chunk from that bin upward joins the row's candidates (in any order), and the chunk's share of Z goes to
// zpart[row][chunk] (zpart may be NULL). The block collects its candidates in LDS and reserves their places in the row's list
// with a single atomic add: a thousand appends to one counter, one by one, would cost more than the rest of the route.
extern "C" __global__ __launch_bounds__(1024) void rd_k_topk_pick(const float *__restrict__ logits, int V, int k, float invT,
                                                                  const float *__restrict__ invTRows, const int *__restrict__ hpart,
                                                                  const uint32_t *__restrict__ mpart, float *__restrict__ cand_v,
                                                                  int *__restrict__ cand_i, int *__restrict__ ccount, double *__restrict__ zpart) {
    __shared__ int tot[RD_TOPK_BINS];
    __shared__ float bval[RD_TOPK_CAP]; // this block's candidates
    __shared__ int bidx[RD_TOPK_CAP];
    __shared__ int s_bin, s_count, s_base;
    __shared__ double wz[16];
    const int t = threadIdx.x, m = blockIdx.y, lane = t & 63, chunks = gridDim.x;
    const float *row = logits + (size_t)m * V;
    const int *hp = hpart + (size_t)m * chunks * RD_TOPK_BINS;
    int a0 = 0, a1 = 0;
    for (int c = 0; c < chunks; c++) a0 += hp[(size_t)c * RD_TOPK_BINS + t], a1 += hp[(size_t)c * RD_TOPK_BINS + 1024 + t];
    tot[t] = a0, tot[1024 + t] = a1;
    uint32_t gk = 0u;
    for (int c = 0; c < chunks; c++) gk = max(gk, mpart[(size_t)m * chunks + c]);
    if (t == 0) s_count = 0;
    __syncthreads();
    if (t < 64) { // the highest bin b with count(bins >= b) >= k: lane l owns bins 32l..32l+31, a suffix scan over the lanes finds the owner
        int own = 0;
        for (int j = 0; j < 32; j++) own += tot[t * 32 + j];
        int above = own; // inclusive suffix sum over lanes >= l
        for (int o = 1; o < 64; o <<= 1) {
            const int v = __shfl_down(above, o, 64);
            if (lane + o < 64) above += v;
        }
        const bool mine = above >= k && above - own < k; // exactly one lane: the counts above it fall short, with its own they reach k
        if (mine) {
            int cum = above - own, b = t * 32 + 31;
            for (; b > t * 32; b--) {
                if (cum + tot[b] >= k) break;
                cum += tot[b];
            }
            s_bin = b;
        }
    }
    __syncthreads();
    const uint32_t bin = (uint32_t)s_bin;
    const float mx = topk_unkey(gk);
    if (invTRows) invT = invTRows[m];
    double acc = 0.0;
    const int base = blockIdx.x * RD_TOPK_CHUNK;
    for (int j = 0; j < RD_TOPK_CHUNK / 1024; j++) {
        const int i = base + j * 1024 + t;
        bool take = false;
        float xv = 0.f;
        if (i < V) {
            const float x = row[i];
            if (zpart) acc += topk_z_term(x, mx, invT);
            take = (topk_key(x) >> 21) >= bin;
            xv = x;
        }
        const unsigned long long mk = __ballot(take); // one LDS append per wave: its lanes' places follow from the ballot
        if (mk) {
            const int first = __ffsll((long long)mk) - 1;
            int p0 = 0;
            if (lane == first) p0 = atomicAdd(&s_count, __popcll(mk));
            p0 = __shfl(p0, first, 64);
            const int p = p0 + __popcll(mk & ((1ull << lane) - 1ull));
            if (take && p < RD_TOPK_CAP) bval[p] = xv, bidx[p] = i;
        }
    }
    __syncthreads();
    const int n = s_count; // may exceed the list: then the row's count does too, and the last launch takes the exact route
    if (t == 0) s_base = n ? atomicAdd(ccount + m, n) : 0;
    __syncthreads();
    const int gb = s_base;
    for (int p = t; p < min(n, RD_TOPK_CAP); p += 1024)
        if (gb + p < RD_TOPK_CAP) cand_v[(size_t)m * RD_TOPK_CAP + gb + p] = bval[p], cand_i[(size_t)m * RD_TOPK_CAP + gb + p] = bidx[p];
    if (zpart) {
        for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
        if (lane == 0) wz[t >> 6] = acc;
        __syncthreads();
        if (t == 0) {
            double z = 0.0;
            for (int w = 0; w < 16; w++) z += wz[w];
            zpart[(size_t)m * chunks + blockIdx.x] = z;
        }
    }
}

// Grid (rows), block 1024: the candidates sorted and cut to k — or, when they overflowed the list, the exact route over the row —
// then Z from the chunks' shares in chunk order, and the row's candidate count back to zero.
extern "C" __global__ __launch_bounds__(RD_TOPK_THREADS) void rd_k_topk_finish(const float *__restrict__ logits, int V, int k, int chunks,
                                                                               const float *__restrict__ cand_v, const int *__restrict__ cand_i,
                                                                               int *__restrict__ ccount, const double *__restrict__ zpart,
                                                                               int *__restrict__ ids_out, float *__restrict__ vals_out,
                                                                               double *__restrict__ z_out) {
    __shared__ TopkShared sh;
    const int t = threadIdx.x, m = blockIdx.x;
    const int C = ccount[m];
    if (C <= RD_TOPK_CAP) {
        for (int i = t; i < C; i += RD_TOPK_THREADS) sh.sval[i] = cand_v[(size_t)m * RD_TOPK_CAP + i], sh.sidx[i] = cand_i[(size_t)m * RD_TOPK_CAP + i];
        __syncthreads();
        topk_sort(sh, C);
    } else {
        topk_select_exact(logits + (size_t)m * V, V, k, sh);
        topk_sort(sh, k);
    }
    for (int i = t; i < k; i += RD_TOPK_THREADS) ids_out[(size_t)m * k + i] = sh.sidx[i], vals_out[(size_t)m * k + i] = sh.sval[i];
    if (z_out && t == 0) {
        double z = 0.0;
        for (int c = 0; c < chunks; c++) z += zpart[(size_t)m * chunks + c];
        z_out[m] = z;
    }
    __syncthreads(); // every thread has read ccount
    if (t == 0) ccount[m] = 0;
}
