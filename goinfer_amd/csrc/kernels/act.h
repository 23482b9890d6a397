// act.h — the row-wise glue between GEMMs: split-K reduction, residual add, RMSNorm, SwiGLU, and the int8 activation quantization
// (per group of 32, or per row) written in the layout the next GEMM reads.
#pragma once
#include "a8.h"
#include "common.h"

// Activation layouts: A8 blocks for the int8-MFMA GEMMs (a8.h), ROW8 plain rows for the experts' vector-ALU kernels.
enum { RD_PANEL_A8 = 3, RD_PANEL_ROW8 = 4 };

// One quantized element: its int8 code, the group's scale and scaled code sum, and the dequantized value code * scale that
// the f16 panel kinds store.
struct Quant1 {
    int code;
    float sc, gsum, xhat;
};
__device__ __forceinline__ Quant1 quant_one(float v) { // an aligned half-wave holds one group of 32
    Quant1 q;
    q.code = quant8_g32(v, &q.sc, &q.gsum);
    q.xhat = __fmul_rn((float)q.code, q.sc);
    return q;
}
// Four consecutive elements per lane (a group is 8 consecutive lanes).
struct Quant4 {
    uint32_t codes; // packed, low byte first
    float sc, gsum, x[4];
};
__device__ __forceinline__ Quant4 quant_four(float v0, float v1, float v2, float v3) {
    Quant4 q;
    q.codes = quant8_g32x4(v0, v1, v2, v3, &q.sc, &q.gsum);
#pragma unroll
    for (int i = 0; i < 4; i++) q.x[i] = __fmul_rn((float)(int)(signed char)(q.codes >> (8 * i)), q.sc);
    return q;
}

// The same against a scale that belongs to the whole row (ActQuantGroup 0).
__device__ __forceinline__ Quant4 quant_four_row(float v0, float v1, float v2, float v3, float s) {
    Quant4 q;
    q.sc = s;
    q.codes = quant8_rowx4(v0, v1, v2, v3, s, &q.gsum);
#pragma unroll
    for (int i = 0; i < 4; i++) q.x[i] = __fmul_rn((float)(int)(signed char)(q.codes >> (8 * i)), q.sc);
    return q;
}
// The maximum of v over a block of up to 1024 threads, on every thread. red: 16 floats of LDS; every thread calls it.
__device__ __forceinline__ float block_max(float v, float *red) {
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    __syncthreads(); // red may still be read from an earlier call
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float m = 0.f;
    for (int i = 0; i < (int)((blockDim.x + 63) >> 6); i++) m = fmaxf(m, red[i]);
    return m;
}

// Store one quantized activation (element k of batch row m) in the layout the consuming GEMM reads. ldk: the row length, for
// the one layout that needs it (RD_PANEL_ROW8).
__device__ __forceinline__ void panel_store(uint8_t *__restrict__ Xp, int kind, int m, int k, const Quant1 &q, int ldk = 0) {
    if (kind == RD_PANEL_ROW8) {
        row8_store1(Xp, ldk, m, k, q.code, q.sc, q.gsum);
    } else {
        Xp[a8_code_offset(m, k)] = (uint8_t)q.code;
        if ((k & 31) == 0) {
            uint8_t *p = Xp + a8_scale_offset(m, k >> 5);
            *(float *)p = q.sc;
            *(float *)(p + (RD_A8_SUMS - RD_A8_SCALES)) = q.gsum;
        }
    }
}

// Four consecutive elements k0..k0+3 (k0 % 4 == 0) of batch row m.
__device__ __forceinline__ void panel_store4(uint8_t *__restrict__ Xp, int kind, int m, int k0, const Quant4 &q, int ldk = 0) {
    if (kind == RD_PANEL_ROW8) {
        row8_store4(Xp, ldk, m, k0, q.codes, q.sc, q.gsum);
    } else {
        a8_store4(Xp, m, k0, q.codes, q.sc, q.gsum);
    }
}

// x f32 [M][K] -> panels. Grid (K/256, M), 256 threads: thread t is element t of the 256-wide chunk.
extern "C" __global__ __launch_bounds__(256) void rd_k_quant_act(const float *__restrict__ x, uint8_t *__restrict__ Xp, int K, int kind) {
    int m = blockIdx.y, k = blockIdx.x * 256 + threadIdx.x;
    float v = k < K ? x[(size_t)m * K + k] : 0.f;
    const Quant1 q = quant_one(v);
    if (k < K || kind == RD_PANEL_A8) panel_store(Xp, kind, m, k, q); // A8: the tail of the last block is written as zero groups
}

// The same with one scale per row (ActQuantGroup 0: linalg.QuantizeRowInt8; the scale lands in every group's slot of the row, the
// sums stay per group of 32). Grid (M), 1024 threads, four consecutive elements per thread and round; K % 32 == 0. The row is
// read twice: once for its maximum, once for its codes.
extern "C" __global__ __launch_bounds__(1024) void rd_k_quant_act_row(const float *__restrict__ x, uint8_t *__restrict__ Xp, int K, int kind) {
    __shared__ float red[16];
    const int m = blockIdx.x, t = threadIdx.x, nv = K >> 2;
    const int nvPad = kind == RD_PANEL_A8 ? ((K + 255) >> 8) << 6 : nv; // A8: the tail of the last block is written as zero codes
    const float *row = x + (size_t)m * K;
    float ma = 0.f;
    for (int q = t; q < nv; q += 1024) {
        const float4_t v = *(const float4_t *)(row + 4 * q);
        ma = fmaxf(ma, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    }
    const float s = row_scale_of(block_max(ma, red));
    for (int q = t; q < nvPad; q += 1024) { // groups of 8 lanes are inside K or past it together
        float4_t v = {0.f, 0.f, 0.f, 0.f};
        if (q < nv) v = *(const float4_t *)(row + 4 * q);
        const Quant4 qq = quant_four_row(v.x, v.y, v.z, v.w, s);
        panel_store4(Xp, kind, m, 4 * q, qq, K);
    }
}

// out[m][n] = sum_s P[s][m][n] in ascending split order (deterministic).
extern "C" __global__ void rd_k_reduce_splits(const float *__restrict__ P, float *__restrict__ out, int N, int splits) {
    int m = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x;
    if (n >= N) return;
    float a = P[(size_t)m * N + n];
    for (int s = 1; s < splits; s++) a = __fadd_rn(a, P[((size_t)s * 32 + m) * N + n]);
    out[(size_t)m * N + n] = a;
}

// One block (1024 threads) per batch row, four consecutive elements per thread:
//   h[m] (+)= sum_s P[s][m][:]   (residual add of a split-K GEMM result, when P != nullptr; ascending split order)
//   normed = (h*inv)*w with inv = f32(1/sqrt(ss/H+eps)), ss summed in f64   (decoder/rmsnorm.go:29-92)
//   panels <- per-32 quantization of normed                                  (weightmat.go:33-38)
// Optionally writes normed f32 to norm_out (the MoE router reads the un-quantized row). H % 128 == 0, H <= 8192.
// foldW != NULL: the pending contribution is an MoE layer's output instead, folded here from the experts' down-projection rows:
// P is [(row*k + rank)][H] with k = splits (<= 8), foldW is [row][k], and the row's contribution is the sum over ranks, in rank
// order from zero, of foldW * P (multiply, then add: decoder/mlp.go:100-103 addScaled).
// postW != NULL (split-K contributions only): the summed contribution x is replaced by (x * invx) * postW, its own RMSNorm with
// the same eps, before the add: Gemma 2's post-attention / post-feed-forward norm (decoder/program_cpu.go:286-312).
extern "C" __global__ __launch_bounds__(1024) void rd_k_add_rmsnorm_quant(float *__restrict__ h, const float *__restrict__ P, int splits,
                                                                          const float *__restrict__ w, float eps, int H,
                                                                          uint8_t *__restrict__ Xp, int kind, float *__restrict__ norm_out,
                                                                          size_t pStride, size_t xpStride, const float *__restrict__ foldW,
                                                                          const float *__restrict__ postW, int actGroup) {
    __shared__ double red[16], redPost[16];
    __shared__ float redMax[16];
    const int m = blockIdx.x, t = threadIdx.x, nv = H >> 2;
    // rows beyond 32 are further M-tiles: their partial sums and panels sit pStride floats / xpStride bytes further on
    const int mt = m >> 5, mr = m & 31;
    if (P) P += (size_t)mt * pStride;
    Xp += (size_t)mt * xpStride;
    float4_t v[2];
    bool on[2];
    double ss = 0;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        int q = t + i * 1024;
        on[i] = q < nv;
        v[i] = (float4_t){0.f, 0.f, 0.f, 0.f};
        if (on[i]) v[i] = *(const float4_t *)(h + (size_t)m * H + 4 * q);
    }
    float4_t wv[2]; // the norm weights are needed last: ask for them first
#pragma unroll
    for (int i = 0; i < 2; i++)
        if (on[i]) wv[i] = *(const float4_t *)(w + 4 * (t + i * 1024));
    if (P && foldW) {
        float4_t b[2][8];
        float wr[8];
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (j < splits) {
                wr[j] = foldW[m * splits + j];
#pragma unroll
                for (int i = 0; i < 2; i++)
                    if (on[i]) b[i][j] = *(const float4_t *)(P + ((size_t)m * splits + j) * H + 4 * (t + i * 1024));
            }
#pragma unroll
        for (int i = 0; i < 2; i++) {
            if (!on[i]) continue;
            float4_t a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < 8; j++)
                if (j < splits) {
                    a.x = __fadd_rn(a.x, mul_rounded(wr[j], b[i][j].x)), a.y = __fadd_rn(a.y, mul_rounded(wr[j], b[i][j].y));
                    a.z = __fadd_rn(a.z, mul_rounded(wr[j], b[i][j].z)), a.w = __fadd_rn(a.w, mul_rounded(wr[j], b[i][j].w));
                }
            v[i].x = __fadd_rn(v[i].x, a.x), v[i].y = __fadd_rn(v[i].y, a.y), v[i].z = __fadd_rn(v[i].z, a.z), v[i].w = __fadd_rn(v[i].w, a.w);
            *(float4_t *)(h + (size_t)m * H + 4 * (t + i * 1024)) = v[i];
        }
    } else if (P) {
        // the split-K partials in ascending split order; eight splits' loads are issued together (a runtime-trip loop of
        // dependent adds would expose one memory latency per split)
        float4_t a[2];
#pragma unroll
        for (int i = 0; i < 2; i++)
            if (on[i]) a[i] = *(const float4_t *)(P + (size_t)mr * H + 4 * (t + i * 1024));
        for (int s0 = 1; s0 < splits; s0 += 8) {
            float4_t b[2][8];
#pragma unroll
            for (int j = 0; j < 8; j++)
#pragma unroll
                for (int i = 0; i < 2; i++)
                    if (on[i] && s0 + j < splits) b[i][j] = *(const float4_t *)(P + ((size_t)(s0 + j) * 32 + mr) * H + 4 * (t + i * 1024));
#pragma unroll
            for (int j = 0; j < 8; j++)
#pragma unroll
                for (int i = 0; i < 2; i++)
                    if (on[i] && s0 + j < splits) {
                        a[i].x = __fadd_rn(a[i].x, b[i][j].x), a[i].y = __fadd_rn(a[i].y, b[i][j].y);
                        a[i].z = __fadd_rn(a[i].z, b[i][j].z), a[i].w = __fadd_rn(a[i].w, b[i][j].w);
                    }
        }
        if (postW) { // the branch output goes through its own RMSNorm before it joins the residual
            double sp = 0;
#pragma unroll
            for (int i = 0; i < 2; i++)
                if (on[i]) sp += (double)a[i].x * a[i].x + (double)a[i].y * a[i].y + (double)a[i].z * a[i].z + (double)a[i].w * a[i].w;
            sp = wave_sum64_d(sp);
            if ((t & 63) == 0) redPost[t >> 6] = sp;
            __syncthreads();
            sp = 0;
#pragma unroll
            for (int i = 0; i < 16; i++) sp += redPost[i];
            const float invP = (float)(1.0 / sqrt(sp / (double)H + (double)eps));
#pragma unroll
            for (int i = 0; i < 2; i++)
                if (on[i]) {
                    const float4_t pw = *(const float4_t *)(postW + 4 * (t + i * 1024));
                    a[i].x = __fmul_rn(__fmul_rn(a[i].x, invP), pw.x), a[i].y = __fmul_rn(__fmul_rn(a[i].y, invP), pw.y);
                    a[i].z = __fmul_rn(__fmul_rn(a[i].z, invP), pw.z), a[i].w = __fmul_rn(__fmul_rn(a[i].w, invP), pw.w);
                }
        }
#pragma unroll
        for (int i = 0; i < 2; i++)
            if (on[i]) {
                v[i].x = __fadd_rn(v[i].x, a[i].x), v[i].y = __fadd_rn(v[i].y, a[i].y), v[i].z = __fadd_rn(v[i].z, a[i].z), v[i].w = __fadd_rn(v[i].w, a[i].w);
                *(float4_t *)(h + (size_t)m * H + 4 * (t + i * 1024)) = v[i];
            }
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
        ss += (double)v[i].x * v[i].x + (double)v[i].y * v[i].y + (double)v[i].z * v[i].z + (double)v[i].w * v[i].w;
    ss = wave_sum64_d(ss);
    if ((t & 63) == 0) red[t >> 6] = ss;
    __syncthreads();
    ss = 0;
#pragma unroll
    for (int i = 0; i < 16; i++) ss += red[i];
    float inv = (float)(1.0 / sqrt(ss / (double)H + (double)eps));
    float4_t nn[2];
    float ma = 0.f;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        nn[i] = (float4_t){0.f, 0.f, 0.f, 0.f};
        if (!on[i]) continue;
        nn[i].x = __fmul_rn(__fmul_rn(v[i].x, inv), wv[i].x), nn[i].y = __fmul_rn(__fmul_rn(v[i].y, inv), wv[i].y);
        nn[i].z = __fmul_rn(__fmul_rn(v[i].z, inv), wv[i].z), nn[i].w = __fmul_rn(__fmul_rn(v[i].w, inv), wv[i].w);
        ma = fmaxf(ma, fmaxf(fmaxf(fabsf(nn[i].x), fabsf(nn[i].y)), fmaxf(fabsf(nn[i].z), fabsf(nn[i].w))));
    }
    // actGroup 0: the consuming projections take one activation scale per row (linalg.QuantizeRowInt8) instead of one per 32
    const float rowS = actGroup == 0 ? row_scale_of(block_max(ma, redMax)) : 0.f;
#pragma unroll
    for (int i = 0; i < 2; i++) {
        if (!on[i]) continue; // whole waves drop out together: nv is a multiple of 32
        int k0 = 4 * (t + i * 1024);
        const float n0 = nn[i].x, n1 = nn[i].y, n2 = nn[i].z, n3 = nn[i].w;
        if (norm_out) *(float4_t *)(norm_out + (size_t)m * H + k0) = nn[i];
        const Quant4 q = actGroup == 0 ? quant_four_row(n0, n1, n2, n3, rowS) : quant_four(n0, n1, n2, n3);
        panel_store4(Xp, kind, mr, k0, q, H);
    }
}

// What rd_k_add_rmsnorm_quant leaves for ONE row (row 0 of a one-row step), recomputed by every block of the projection that
// consumes it instead of being its own launch: a step of one sequence is bound by its launches, and the row is 16 KB. The plain
// case only: split-K partials (or none), one scale per group of 32, no second norm, H % 256 == 0, H <= 4096. The block's BS
// threads stand in for the standalone kernel's 1024: thread t is its threads t, t + BS, ... (same lane, so the wave sums and the
// eight-lane quantization groups are the same lanes' — the same operations on the same values, bit for bit).
//   hOut (every block holds the same values; the caller lets one block pass it): the residual row after the add
//   img: the row's quantized form in LDS, RD_ROW0_KB_BYTES per 256 elements: codes [8 groups][32], then the groups' scales as
//        [parity][4] floats and their scaled code sums alike — a lane half's sixteen codes of a group, and the scales and sums of
//        its parity's four groups, are one 16-byte read each (a8_row0_from_lds)
//   red: 16 doubles of LDS. Ends with a barrier: img is complete when it returns.
constexpr int RD_ROW0_KB_BYTES = 320;
template <int BS>
__device__ __forceinline__ void norm_row0_to_lds(const float *__restrict__ hIn, float *__restrict__ hOut, const float *__restrict__ P, int splits,
                                                 const float *__restrict__ w, float eps, int H, uint8_t *img, double *red) {
    constexpr int NV = 1024 / BS;
    const int t = threadIdx.x, nv = H >> 2;
    float4_t v[NV], wv[NV], a[NV];
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int q = t + j * BS;
        v[j] = (float4_t){0.f, 0.f, 0.f, 0.f};
        if (q < nv) v[j] = *(const float4_t *)(hIn + 4 * q), wv[j] = *(const float4_t *)(w + 4 * q);
        if (q < nv && P) a[j] = *(const float4_t *)(P + 4 * q);
    }
    if (P) {
        for (int s = 1; s < splits; s++) // ascending split order
#pragma unroll
            for (int j = 0; j < NV; j++) {
                const int q = t + j * BS;
                if (q >= nv) continue;
                const float4_t b = *(const float4_t *)(P + (size_t)s * 32 * H + 4 * q);
                a[j].x = __fadd_rn(a[j].x, b.x), a[j].y = __fadd_rn(a[j].y, b.y), a[j].z = __fadd_rn(a[j].z, b.z), a[j].w = __fadd_rn(a[j].w, b.w);
            }
#pragma unroll
        for (int j = 0; j < NV; j++)
            if (t + j * BS < nv)
                v[j].x = __fadd_rn(v[j].x, a[j].x), v[j].y = __fadd_rn(v[j].y, a[j].y), v[j].z = __fadd_rn(v[j].z, a[j].z), v[j].w = __fadd_rn(v[j].w, a[j].w);
    }
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int q = t + j * BS;
        if (hOut && q < nv) *(float4_t *)(hOut + 4 * q) = v[j];
        double ss = 0;
        ss += (double)v[j].x * v[j].x + (double)v[j].y * v[j].y + (double)v[j].z * v[j].z + (double)v[j].w * v[j].w;
        ss = wave_sum64_d(ss);
        if ((t & 63) == 0) red[q >> 6] = ss;
    }
    __syncthreads();
    double ss = 0;
#pragma unroll
    for (int i = 0; i < 16; i++) ss += red[i];
    const float inv = (float)(1.0 / sqrt(ss / (double)H + (double)eps));
#pragma unroll
    for (int j = 0; j < NV; j++) {
        const int q = t + j * BS;
        if (q >= nv) continue; // whole waves drop out together: nv is a multiple of 64
        const float n0 = __fmul_rn(__fmul_rn(v[j].x, inv), wv[j].x), n1 = __fmul_rn(__fmul_rn(v[j].y, inv), wv[j].y);
        const float n2 = __fmul_rn(__fmul_rn(v[j].z, inv), wv[j].z), n3 = __fmul_rn(__fmul_rn(v[j].w, inv), wv[j].w);
        const Quant4 qq = quant_four(n0, n1, n2, n3);
        const int k0 = 4 * q, g = (k0 >> 5) & 7;
        uint8_t *kb = img + (size_t)(k0 >> 8) * RD_ROW0_KB_BYTES;
        *(uint32_t *)(kb + g * 32 + (k0 & 31)) = qq.codes;
        if ((k0 & 31) == 0) {
            *(float *)(kb + 256 + (g & 1) * 16 + (g >> 1) * 4) = qq.sc;
            *(float *)(kb + 288 + (g & 1) * 16 + (g >> 1) * 4) = qq.gsum;
        }
    }
    __syncthreads();
}

// gate/up partials P[s][32][2I] -> act = silu(gate)*up (decoder/rmsnorm.go:204-207: silu in f64) -> per-32 quant -> panels.
// Grid (ceil(I/1024), M), 256 threads, four consecutive columns per thread. I % 32 == 0. act 1: geluTanh(gate)*up (GeGLU).
extern "C" __global__ __launch_bounds__(256) void rd_k_swiglu_quant(const float *__restrict__ P, int splits, int I, uint8_t *__restrict__ Xp,
                                                                    int kind, float *__restrict__ act_out, size_t pStride, size_t xpStride, int act) {
    const int row = blockIdx.y, m = row & 31, n0 = (blockIdx.x * 256 + threadIdx.x) * 4;
    P += (size_t)(row >> 5) * pStride; // M-tile of this row
    Xp += (size_t)(row >> 5) * xpStride;
    bool on = n0 < I; // groups of 8 lanes are on or off together
    float a[4] = {0.f, 0.f, 0.f, 0.f};
    if (on) {
        int N2 = 2 * I;
        float4_t g = *(const float4_t *)(P + (size_t)m * N2 + n0), u = *(const float4_t *)(P + (size_t)m * N2 + I + n0);
        for (int s = 1; s < splits; s++) {
            float4_t g2 = *(const float4_t *)(P + ((size_t)s * 32 + m) * N2 + n0), u2 = *(const float4_t *)(P + ((size_t)s * 32 + m) * N2 + I + n0);
            g.x = __fadd_rn(g.x, g2.x), g.y = __fadd_rn(g.y, g2.y), g.z = __fadd_rn(g.z, g2.z), g.w = __fadd_rn(g.w, g2.w);
            u.x = __fadd_rn(u.x, u2.x), u.y = __fadd_rn(u.y, u2.y), u.z = __fadd_rn(u.z, u2.z), u.w = __fadd_rn(u.w, u2.w);
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            a[i] = __fmul_rn(gate_act(g[i], act), u[i]);
        }
        if (act_out) *(float4_t *)(act_out + (size_t)row * I + n0) = (float4_t){a[0], a[1], a[2], a[3]};
    }
    const Quant4 q = quant_four(a[0], a[1], a[2], a[3]);
    if (on) panel_store4(Xp, kind, m, n0, q);
}

// The same with one scale per row of I (ActQuantGroup 0). Grid (M), 1024 threads: a thread keeps up to eight groups of four
// columns (I <= 32768, I % 32 == 0) in registers between the row's maximum and its codes.
extern "C" __global__ __launch_bounds__(1024) void rd_k_swiglu_quant_row(const float *__restrict__ P, int splits, int I, uint8_t *__restrict__ Xp,
                                                                         int kind, size_t pStride, size_t xpStride, int act) {
    __shared__ float red[16];
    const int row = blockIdx.x, m = row & 31, t = threadIdx.x, nv = I >> 2, N2 = 2 * I;
    P += (size_t)(row >> 5) * pStride;
    Xp += (size_t)(row >> 5) * xpStride;
    float4_t a[8];
    float ma = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int q = t + i * 1024;
        a[i] = (float4_t){0.f, 0.f, 0.f, 0.f};
        if (q >= nv) continue;
        const int n0 = 4 * q;
        float4_t g = *(const float4_t *)(P + (size_t)m * N2 + n0), u = *(const float4_t *)(P + (size_t)m * N2 + I + n0);
        for (int s = 1; s < splits; s++) {
            float4_t g2 = *(const float4_t *)(P + ((size_t)s * 32 + m) * N2 + n0), u2 = *(const float4_t *)(P + ((size_t)s * 32 + m) * N2 + I + n0);
            g.x = __fadd_rn(g.x, g2.x), g.y = __fadd_rn(g.y, g2.y), g.z = __fadd_rn(g.z, g2.z), g.w = __fadd_rn(g.w, g2.w);
            u.x = __fadd_rn(u.x, u2.x), u.y = __fadd_rn(u.y, u2.y), u.z = __fadd_rn(u.z, u2.z), u.w = __fadd_rn(u.w, u2.w);
        }
#pragma unroll
        for (int e = 0; e < 4; e++) a[i][e] = __fmul_rn(gate_act(g[e], act), u[e]);
        ma = fmaxf(ma, fmaxf(fmaxf(fabsf(a[i].x), fabsf(a[i].y)), fmaxf(fabsf(a[i].z), fabsf(a[i].w))));
    }
    const float s = row_scale_of(block_max(ma, red));
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int q = t + i * 1024;
        if (q >= nv) continue; // groups of 8 lanes are on or off together
        const Quant4 qq = quant_four_row(a[i].x, a[i].y, a[i].z, a[i].w, s);
        panel_store4(Xp, kind, m, 4 * q, qq, I);
    }
}
