// misc.h — small row-wise kernels: plain RMSNorm and RoPE (kernel-level entry points), argmax, the f32 matmul behind
// Backend.MatmulBT / the MoE router, and MoE routing.
#pragma once
#include "common.h"

// decoder/rmsnorm.go:29-92. One block (256 threads) per row; H <= 8192.
extern "C" __global__ __launch_bounds__(256) void rd_k_rmsnorm(const float *__restrict__ x, const float *__restrict__ w, float *__restrict__ out,
                                                               int H, float eps) {
    __shared__ double red[4];
    int m = blockIdx.x, t = threadIdx.x;
    double ss = 0;
    for (int k = t; k < H; k += 256) {
        double v = x[(size_t)m * H + k];
        ss += v * v;
    }
    ss = wave_sum64_d(ss);
    if ((t & 63) == 0) red[t >> 6] = ss;
    __syncthreads();
    ss = (red[0] + red[1]) + (red[2] + red[3]);
    float inv = (float)(1.0 / sqrt(ss / (double)H + (double)eps));
    for (int k = t; k < H; k += 256) out[(size_t)m * H + k] = __fmul_rn(__fmul_rn(x[(size_t)m * H + k], inv), w[k]);
}

// decoder/rope.go:28-64 (NeoX rotate-half, f64 angle and rotation). Grid (heads, rows), block HD/2.
extern "C" __global__ void rd_k_rope(float *__restrict__ vec, const int *__restrict__ pos, const double *__restrict__ invFreq, int heads, int HD) {
    int h = blockIdx.x, m = blockIdx.y, t = threadIdx.x, half = HD / 2;
    float *v = vec + ((size_t)m * heads + h) * HD;
    double theta = (double)pos[m] * invFreq[t], c = cos(theta), s = sin(theta);
    double x1 = v[t], x2 = v[t + half];
    v[t] = (float)(x1 * c - x2 * s);
    v[t + half] = (float)(x2 * c + x1 * s);
}

// Philox4x32-10 (internal/runtime/sampling/philox.go:13-40): integer only, the key bumped between rounds.
__device__ __forceinline__ void philox4x32(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1, uint32_t *out) {
#pragma unroll
    for (int r = 0; r < 10; r++) {
        if (r > 0) k0 += 0x9E3779B9u, k1 += 0xBB67AE85u;
        const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
        const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
        const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
        c0 = n0, c1 = lo1, c2 = n2, c3 = lo0;
    }
    out[0] = c0, out[1] = c1, out[2] = c2, out[3] = c3;
}
// Standard Gumbel variate from 32 random bits, in f64 and rounded once, as the host computes it
// (internal/runtime/sampling/sampler_gumbel.go:33-37): w = (h + 0.5) / 2^32, G = -ln(-ln1p(-w)).
__device__ __forceinline__ float gumbel_noise(uint32_t h) {
    double w = ((double)h + 0.5) * (1.0 / 4294967296.0);
    return (float)(-log(-log1p(-w)));
}

// Per-row draw record, six ints: mode (0 none, 1 greedy, 2 Gumbel-max), 1/T as f32 bits, Philox key (seed lo, hi), draw lo, hi.
#define RD_DRAW_INTS 6

// internal/runtime/sampling/sampler.go:485-520: the first maximum wins. Two stages: per (row, 4096-column chunk) a block
// reduces split-K partials, optionally writes the logits, and leaves its best (value, lowest index); a second kernel folds the
// chunks of each row. N % 4 == 0. A row whose draw record says Gumbel-max competes with key = f32(logit * 1/T) + G_i instead of
// the logit (sampler_gumbel.go:41-66; backend/cuda/gumbel.cu:72-101): entry i takes word i&3 of Philox(counter (i>>2, draw lo,
// draw hi, 0), key seed), and a thread's four consecutive entries are exactly one Philox call.
extern "C" __global__ __launch_bounds__(256) void rd_k_argmax_rows(const float *__restrict__ P, int splits, int N, float *__restrict__ cand_v,
                                                                   int *__restrict__ cand_i, float *__restrict__ logits_out,
                                                                   const int *__restrict__ rowDraw, size_t pStride, float softcap, float logitMul) {
    __shared__ float bv[4];
    __shared__ int bi[4];
    const int m = blockIdx.y, t = threadIdx.x, nChunks = gridDim.x, mr = m & 31;
    P += (size_t)(m >> 5) * pStride; // rows beyond 32 are further M-tiles of partial sums
    const int *dr = rowDraw ? rowDraw + m * RD_DRAW_INTS : nullptr;
    const bool gumbel = dr && dr[0] == 2;
    const float invT = gumbel ? __int_as_float(dr[1]) : 1.f;
    float best = -INFINITY;
    int idx = 0x7fffffff;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int n0 = blockIdx.x * 4096 + (i * 256 + t) * 4;
        if (n0 < N) {
            float4_t a = *(const float4_t *)(P + (size_t)mr * N + n0);
            for (int s = 1; s < splits; s++) {
                float4_t b = *(const float4_t *)(P + ((size_t)s * 32 + mr) * N + n0);
                a.x = __fadd_rn(a.x, b.x), a.y = __fadd_rn(a.y, b.y), a.z = __fadd_rn(a.z, b.z), a.w = __fadd_rn(a.w, b.w);
            }
            if (softcap > 0.f) { // decoder/model_forward.go:259-266: cap * f32(tanh(f64(logit / cap))), before anything reads the logits
#pragma unroll
                for (int e = 0; e < 4; e++) a[e] = mul_rounded(softcap, (float)tanh((double)__fdiv_rn(a[e], softcap)));
            }
            if (logitMul != 0.f && logitMul != 1.f) { // decoder/model_forward.go:304-320: logits *= f32(1 / LogitScale), after the softcap
#pragma unroll
                for (int e = 0; e < 4; e++) a[e] = mul_rounded(a[e], logitMul);
            }
            if (logits_out) *(float4_t *)(logits_out + (size_t)m * N + n0) = a;
            if (gumbel) {
                uint32_t r[4];
                philox4x32((uint32_t)(n0 >> 2), (uint32_t)dr[4], (uint32_t)dr[5], 0u, (uint32_t)dr[2], (uint32_t)dr[3], r);
#pragma unroll
                for (int e = 0; e < 4; e++) a[e] = __fadd_rn(mul_rounded(a[e], invT), gumbel_noise(r[e]));
            }
#pragma unroll
            for (int e = 0; e < 4; e++)
                if (a[e] > best) best = a[e], idx = n0 + e; // ascending n within a thread: strict '>' keeps the lowest index
        }
    }
    for (int o = 32; o > 0; o >>= 1) {
        float v2 = __shfl_xor(best, o, 64);
        int i2 = __shfl_xor(idx, o, 64);
        if (v2 > best || (v2 == best && i2 < idx)) best = v2, idx = i2;
    }
    if ((t & 63) == 0) bv[t >> 6] = best, bi[t >> 6] = idx;
    __syncthreads();
    if (t == 0) {
        for (int w = 1; w < 4; w++)
            if (bv[w] > best || (bv[w] == best && bi[w] < idx)) best = bv[w], idx = bi[w];
        cand_v[m * nChunks + blockIdx.x] = best;
        cand_i[m * nChunks + blockIdx.x] = idx;
    }
}

// w[i] = 1 + w[i]: a norm weight stored as its deviation from one (Gemma; decoder/rmsnorm.go:62-75 scales by f32(1 + w)).
extern "C" __global__ void rd_k_add_one(float *__restrict__ w, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) w[i] = __fadd_rn(1.f, w[i]);
}

// Folds a row's chunk candidates. No comparable candidate (every key -Inf or NaN: a fully masked row) gives index 0, which
// is what the plain argmax the host falls back to returns for such a row (sampler_gumbel.go:104-107).
extern "C" __global__ __launch_bounds__(64) void rd_k_argmax_final(const float *__restrict__ cand_v, const int *__restrict__ cand_i, int nChunks,
                                                                   int *__restrict__ ids) {
    const int m = blockIdx.x, t = threadIdx.x;
    float best = -INFINITY;
    int idx = 0x7fffffff;
    for (int c = t; c < nChunks; c += 64) {
        float v = cand_v[m * nChunks + c];
        int i = cand_i[m * nChunks + c];
        if (v > best || (v == best && i < idx)) best = v, idx = i;
    }
    for (int o = 32; o > 0; o >>= 1) {
        float v2 = __shfl_xor(best, o, 64);
        int i2 = __shfl_xor(idx, o, 64);
        if (v2 > best || (v2 == best && i2 < idx)) best = v2, idx = i2;
    }
    if (t == 0) ids[m] = idx == 0x7fffffff ? 0 : idx;
}

// dst[M][N] = a[M][K] . b[N][K]^T accumulated in f64 and rounded once: Backend.MatmulBT (decoder/backend.go:26-30) and the
// f32 MoE router (decoder/mlp.go:50). One wave per output: each lane sums its share of k in f64, then a fixed butterfly adds the
// 64 lane sums. Products of two f32 are exact in f64 and the sum carries ~29 spare bits, so the f32 result matches an
// ascending-k f64 sum except when that sum falls within ~1e-15 (relative) of an f32 rounding boundary.
// Grid (ceil(N/4), M), block 256. clear8 (may be NULL): eight words this launch sets to zero on the side — the router's launch
// clears the active-expert bitmap that the routing kernel, next in the stream, fills; clearN (may be NULL): nClear more words
// (the experts' row maxima, which the gate|up kernel of the same layer accumulates with atomics).
extern "C" __global__ __launch_bounds__(256) void rd_k_matmul_f32(const float *__restrict__ a, const float *__restrict__ b, float *__restrict__ dst,
                                                                   int M, int K, int N, unsigned *__restrict__ clear8, unsigned *__restrict__ clearN,
                                                                   int nClear) {
    if (clear8 && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x < 8) clear8[threadIdx.x] = 0u;
    if (clearN && blockIdx.x == 0 && blockIdx.y == 0)
        for (int i = threadIdx.x; i < nClear; i += 256) clearN[i] = 0u;
    const int lane = threadIdx.x & 63, n = blockIdx.x * 4 + (threadIdx.x >> 6), m = blockIdx.y;
    if (n >= N || m >= M) return;
    const float *ar = a + (size_t)m * K, *br = b + (size_t)n * K;
    double acc = 0;
    if ((K & 255) == 0) { // 16-byte loads, eight in flight per operand
        const float4_t *a4 = (const float4_t *)ar + lane, *b4 = (const float4_t *)br + lane;
        for (int c0 = 0; c0 < K / 256; c0 += 8) {
            float4_t av[8], bv[8];
#pragma unroll
            for (int c = 0; c < 8; c++)
                if (c0 + c < K / 256) av[c] = a4[(c0 + c) * 64], bv[c] = b4[(c0 + c) * 64];
#pragma unroll
            for (int c = 0; c < 8; c++)
                if (c0 + c < K / 256) {
                    acc = fma((double)av[c].x, (double)bv[c].x, acc);
                    acc = fma((double)av[c].y, (double)bv[c].y, acc);
                    acc = fma((double)av[c].z, (double)bv[c].z, acc);
                    acc = fma((double)av[c].w, (double)bv[c].w, acc);
                }
        }
    } else {
        for (int k = lane; k < K; k += 64) acc = fma((double)ar[k], (double)br[k], acc);
    }
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
    if (lane == 0) dst[(size_t)m * N + n] = (float)acc;
}

// decoder/mlp.go:130-228 routeExperts / groupLimit + mlp.go:370-440 softmaxF32 / topK.
// Scores: softmax (f32 max; e = f32(exp(f64(x - max))); f64 sum in ascending expert order; scores *= f32(1/sum)) or, for the
// DeepSeek / GLM routers, each expert's own f32(1 / (1 + exp(-f64(x)))). Selection scores: scores + bias where the layer has an
// e_score_correction_bias; with nGroup > 1 only the experts of the topkGroup best groups stay eligible (a group's score: the sum
// of its two largest selection scores), the others become -inf and are never chosen. k passes of strict '>' (lowest index wins).
// Weights: the chosen experts' unbiased scores, optionally divided by their f32 sum in rank order, then times scale when that
// is neither 0 nor 1.
// One wave per token (nE <= 256: up to four experts per lane). The f64 sum is taken by every lane over the same ascending
// sequence (from LDS), so it is the reference's sum bit for bit. Also fills rankOf[token][expert] = rank or -1 for the
// expert-major grouped GEMMs. Grid (T), block 64.
struct RouteOpts {
    const float *bias; // [nE] or NULL
    int sigmoid;
    float scale; // 0 or 1: none
    int nGroup, topkGroup; // nGroup <= 32
};
// a key that orders as the floats do (-0 and +0 alike), 0 for "nothing": -inf, which topK never picks, and lanes past nE
__device__ __forceinline__ unsigned route_key(float v) {
    if (!(v > -INFINITY)) return 0u;
    if (v == 0.f) v = 0.f;
    const unsigned u = __float_as_uint(v);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
// The routing of one token by one wave (see rd_k_moe_route); x: the token's nE logits (global or LDS). e64: 256 doubles of LDS.
// NJ: experts per lane, nE <= 64 * NJ (the f64 exponentials are the wave's longest chain: a lane computes only those it holds).
template <int NJ>
__device__ __forceinline__ void moe_route_wave(const float *x, int t, int nE, int k, int norm, int *__restrict__ idx, float *__restrict__ wgt,
                                               signed char *__restrict__ rankOf, double *e64, int *__restrict__ idx_copy,
                                               unsigned *__restrict__ activeBits, const RouteOpts &ro) {
    const int lane = threadIdx.x & 63;
    float xv[NJ], sc[NJ], sel[NJ];
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        int i = lane + 64 * j;
        xv[j] = i < nE ? x[i] : -INFINITY;
    }
    if (ro.sigmoid) {
#pragma unroll
        for (int j = 0; j < NJ; j++) sc[j] = (float)(1.0 / (1.0 + exp(-(double)xv[j])));
    } else {
        float mx = xv[0];
#pragma unroll
        for (int j = 1; j < NJ; j++) mx = fmaxf(mx, xv[j]);
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            int i = lane + 64 * j;
            double e = i < nE ? exp((double)__fsub_rn(xv[j], mx)) : 0.0;
            sc[j] = (float)e;
            e64[i] = e; // all 64 * NJ entries: zeros past nE, which leave the sum as it is
        }
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0): this wave's LDS writes have landed before its lanes read them back
        double sum = 0;
        for (int i = 0; i < nE; i += 8) { // eight reads in flight, then the adds in ascending order
            double v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = e64[i + u];
#pragma unroll
            for (int u = 0; u < 8; u++) sum += v[u];
        }
        const float inv = (float)(1.0 / sum);
#pragma unroll
        for (int j = 0; j < NJ; j++) sc[j] = mul_rounded(sc[j], inv); // rounded before a bias is added
    }
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        int i = lane + 64 * j;
        sel[j] = i < nE ? (ro.bias ? __fadd_rn(sc[j], ro.bias[i]) : sc[j]) : -INFINITY;
        if (rankOf && i < nE) rankOf[(size_t)t * nE + i] = -1;
    }
    if (ro.nGroup > 1) {
        // group scores through LDS: the selection scores, then one lane per group, then every lane ranks the groups alike
        float *selbuf = (float *)e64, *gs = selbuf + 256;
        const int gsz = nE / ro.nGroup;
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < NJ; j++) selbuf[lane + 64 * j] = sel[j];
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_s_waitcnt(0xc07f);
        if (lane < ro.nGroup) {
            float top1 = -INFINITY, top2 = -INFINITY;
            for (int i = lane * gsz; i < (lane + 1) * gsz; i++) {
                const float v = selbuf[i];
                if (v > top1)
                    top2 = top1, top1 = v;
                else if (v > top2)
                    top2 = v;
            }
            gs[lane] = __fadd_rn(top1, top2);
        }
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_s_waitcnt(0xc07f);
        unsigned keep = 0u;
        for (int r = 0; r < ro.topkGroup; r++) { // topK over the group scores: strict '>', lowest index wins, -inf never
            float best = -INFINITY;
            int bg = -1;
            for (int g = 0; g < ro.nGroup; g++) {
                const float v = gs[g];
                if (!((keep >> g) & 1u) && v > best) best = v, bg = g;
            }
            if (bg < 0) break;
            keep |= 1u << bg;
        }
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int i = lane + 64 * j, g = i / gsz;
            if (g >= ro.nGroup || !((keep >> g) & 1u)) sel[j] = -INFINITY; // outside the kept groups, or past the last whole group
        }
    }
    float s = 0.f, mine = 0.f; // lane j keeps the rank-j weight
    int n = 0;
    for (int r = 0; r < k; r++) {
        // The pass's pick as the maximum of a 64-bit key per lane: (order-preserving key of the selection score, ~index), 0 for
        // nothing left. Of equal scores the lower index has the larger key, which is the strict '>' scan's choice. The maximum
        // over the wave: within rows of 16 lanes on the DPP path, across the rows by swizzle and one permute.
        unsigned kh = 0u, kl = 0u;
#pragma unroll
        for (int j = NJ - 1; j >= 0; j--) { // descending, '>=' on the key: the lowest index among this lane's equals survives
            const unsigned kj = route_key(sel[j]);
            if (kj != 0u && kj >= kh) kh = kj, kl = ~(unsigned)(lane + 64 * j);
        }
        auto take = [&](unsigned oh, unsigned ol) {
            const bool gt = oh > kh || (oh == kh && ol > kl);
            kh = gt ? oh : kh, kl = gt ? ol : kl;
        };
        take((unsigned)dpp_i<RD_DPP_QUAD_XOR1>((int)kh), (unsigned)dpp_i<RD_DPP_QUAD_XOR1>((int)kl));
        take((unsigned)dpp_i<RD_DPP_QUAD_XOR2>((int)kh), (unsigned)dpp_i<RD_DPP_QUAD_XOR2>((int)kl));
        take((unsigned)dpp_i<RD_DPP_HALF_MIRROR>((int)kh), (unsigned)dpp_i<RD_DPP_HALF_MIRROR>((int)kl));
        take((unsigned)dpp_i<RD_DPP_ROW_MIRROR>((int)kh), (unsigned)dpp_i<RD_DPP_ROW_MIRROR>((int)kl));
        take((unsigned)swz_xor16_i((int)kh), (unsigned)swz_xor16_i((int)kl));
        take((unsigned)__shfl_xor((int)kh, 32, 64), (unsigned)__shfl_xor((int)kl, 32, 64));
        if (kh == 0u) break; // nothing left (k > the eligible experts)
        const int bi = (int)~kl, bj = bi >> 6;
        // the weight is the chosen expert's unbiased score, which its own lane holds
        float mineSc = sc[0];
#pragma unroll
        for (int j = 1; j < NJ; j++) mineSc = bj == j ? sc[j] : mineSc;
        const float best = __shfl(mineSc, bi & 63, 64);
#pragma unroll
        for (int j = 0; j < NJ; j++)
            if (bi == lane + 64 * j) {
                sel[j] = -INFINITY; // used
                if (rankOf) rankOf[(size_t)t * nE + bi] = (signed char)r;
            }
        if (lane == r) mine = best;
        if (lane == 0) {
            idx[(size_t)t * k + r] = bi;
            if (idx_copy) idx_copy[(size_t)t * k + r] = bi;
            if (activeBits) atomicOr(activeBits + (bi >> 5), 1u << (bi & 31));
        }
        s = __fadd_rn(s, best);
        n++;
    }
    if (lane < n) {
        float w = (norm && s > 0.f) ? mine / s : mine;
        if (ro.scale != 0.f && ro.scale != 1.f) w = __fmul_rn(w, ro.scale);
        wgt[(size_t)t * k + lane] = w;
    }
}

// idx_copy (may be NULL) receives a second copy of the indices: the step's per-layer routing trace. activeBits (may be NULL):
// a bitmap of nE bits, zero on entry, in which every chosen expert's bit is set.
// bias (may be NULL), sigmoid, scale, nGroup, topkGroup: the router's variant (see above); all zero = softmax top-k.
extern "C" __global__ __launch_bounds__(64) void rd_k_moe_route(const float *__restrict__ logits, int T, int nE, int k, int norm,
                                                                 int *__restrict__ idx, float *__restrict__ wgt, signed char *__restrict__ rankOf,
                                                                 int *__restrict__ idx_copy, unsigned *__restrict__ activeBits,
                                                                 const float *__restrict__ bias, int sigmoid, float scale, int nGroup, int topkGroup) {
    __shared__ double e64[256];
    const int t = blockIdx.x;
    if (t >= T) return;
    const RouteOpts ro{bias, sigmoid, scale, nGroup, topkGroup};
    const float *x = logits + (size_t)t * nE;
    if (nE <= 64)
        moe_route_wave<1>(x, t, nE, k, norm, idx, wgt, rankOf, e64, idx_copy, activeBits, ro);
    else if (nE <= 128)
        moe_route_wave<2>(x, t, nE, k, norm, idx, wgt, rankOf, e64, idx_copy, activeBits, ro);
    else
        moe_route_wave<4>(x, t, nE, k, norm, idx, wgt, rankOf, e64, idx_copy, activeBits, ro);
}

// Token embedding rows from an int8 table with one f32 scale per row (goinfer keeps the embedding table int8 in q4k mode,
// decoder/weightmat.go:79-84; Embed.Row widens q*scale): h[m][k] = q[ids[m]][k] * scale[ids[m]]. Grid (rows), block 256.
extern "C" __global__ void rd_k_embed_rows(const signed char *__restrict__ q, const float *__restrict__ scale, const int *__restrict__ ids,
                                           float *__restrict__ h, int H) {
    int m = blockIdx.x, id = ids[m];
    float sc = scale[id];
    for (int k = threadIdx.x; k < H; k += blockDim.x) h[(size_t)m * H + k] = __fmul_rn((float)q[(size_t)id * H + k], sc);
}

// Plain copy of n16 16-byte words (grid-stride). A traffic yardstick of known size: n16*16 bytes read, n16*16 written.
extern "C" __global__ void rd_k_copy16(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n16) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (size_t)gridDim.x * blockDim.x) dst[i] = src[i];
}

// Issue-rate probes: what one SIMD sustains of the instruction mix of the int8 GEMMs' inner loop, with no memory in the loop. One
// iteration is one (32 x 32 outputs, 256 deep) tile-block's worth: MODE 0 its eight int8 MFMAs, 1 its eight f32 MFMAs (four
// 32x32x1 two-block scale products, four 32x32x2 minimum terms), 2 the fold's 256 vector instructions (128 converts, 128 fmas),
// 3 all of them, none depending on another's result. Launched with (compute units x w) blocks of four waves, every SIMD holds w
// waves; time per launch / iterations / w is the SIMD's time per tile-block. in: 1024 ints; out: one float per thread.
typedef int rd_i32x4_t __attribute__((ext_vector_type(4)));
typedef int rd_i32x16_t __attribute__((ext_vector_type(16)));
typedef float rd_f32x32_t __attribute__((ext_vector_type(32)));
template <int MODE> __device__ __forceinline__ void issue_probe(int iters, const int *__restrict__ in, float *__restrict__ out) {
    const int lane = threadIdx.x & 63;
    const rd_i32x4_t a = {in[lane], in[lane + 64], in[lane + 128], in[lane + 192]};
    const rd_i32x4_t b = {in[lane + 1], in[lane + 65], in[lane + 129], in[lane + 193]};
    const float sa = (float)in[lane + 2] * 1e-3f, sb = (float)in[lane + 3] * 1e-3f;
    float16_t acc = {0.f}, facc = {0.f};
    rd_i32x16_t d0 = {0}, d1 = {0}, p0, p1;
    rd_f32x32_t s2 = {0.f}, ps;
    for (int j = 0; j < 16; j++) p0[j] = in[lane + j], p1[j] = in[lane + j + 7];
    for (int j = 0; j < 32; j++) ps[j] = (float)in[lane + j] * 1e-4f;
    for (int it = 0; it < iters; it++) {
        if (MODE == 0 || MODE == 3) {
#pragma unroll
            for (int p = 0; p < 4; p++) {
                d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, d0, 0, 0, 0);
                d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(b, a, d1, 0, 0, 0);
            }
        }
        if (MODE == 1 || MODE == 3) {
#pragma unroll
            for (int p = 0; p < 4; p++) s2 = __builtin_amdgcn_mfma_f32_32x32x1f32(sa, sb, s2, 0, 0, 0);
#pragma unroll
            for (int p = 0; p < 4; p++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(sa, sb, acc, 0, 0, 0);
        }
        if (MODE == 2 || MODE == 3) {
#pragma unroll
            for (int p = 0; p < 4; p++) {
#pragma unroll
                for (int j = 0; j < 16; j++) {
                    asm volatile("" : "+v"(p0[j])); // the compiler may not hoist the convert out of the loop
                    facc[j] = __builtin_fmaf((float)p0[j], ps[j], facc[j]);
                }
#pragma unroll
                for (int j = 0; j < 16; j++) {
                    asm volatile("" : "+v"(p1[j]));
                    facc[j] = __builtin_fmaf((float)p1[j], ps[16 + j], facc[j]);
                }
            }
        }
    }
    float s = 0.f;
    for (int j = 0; j < 16; j++) s += acc[j] + facc[j] + (float)d0[j] + (float)d1[j] + s2[j] + s2[j + 16];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = s;
}
extern "C" __global__ __launch_bounds__(256) void rd_k_issue_mfma_i8(int iters, const int *in, float *out) { issue_probe<0>(iters, in, out); }
extern "C" __global__ __launch_bounds__(256) void rd_k_issue_mfma_f32(int iters, const int *in, float *out) { issue_probe<1>(iters, in, out); }
extern "C" __global__ __launch_bounds__(256) void rd_k_issue_valu(int iters, const int *in, float *out) { issue_probe<2>(iters, in, out); }
extern "C" __global__ __launch_bounds__(256) void rd_k_issue_all(int iters, const int *in, float *out) { issue_probe<3>(iters, in, out); }

// Synthetic operand fills for the micro-benchmarks: element i = uniform in [-2, 2) from a counter hash of (seed, i).
__device__ __forceinline__ float fill_value(size_t i, unsigned seed) {
    unsigned long long z = (unsigned long long)i * 0x9E3779B97F4A7C15ull + (unsigned long long)seed * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (float)(unsigned)(z >> 40) * (4.0f / 16777216.0f) - 2.0f;
}
extern "C" __global__ void rd_k_fill_f16(uint16_t *__restrict__ dst, size_t n, unsigned seed) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        half_t h = (half_t)fill_value(i, seed);
        uint16_t u;
        __builtin_memcpy(&u, &h, 2);
        dst[i] = u;
    }
}
extern "C" __global__ void rd_k_fill_f32(float *__restrict__ dst, size_t n, unsigned seed) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) dst[i] = fill_value(i, seed);
}
