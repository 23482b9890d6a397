// act.h — the row-wise glue between GEMMs: split-K reduction, residual add, RMSNorm, SwiGLU, and the per-32 int8
// activation quantization whose dequantized values are written as f16 MFMA panels for the next GEMM.
#pragma once
#include "common.h"

enum { RD_PANEL_Q4K = 0, RD_PANEL_LIN = 1, RD_PANEL_LIN4 = 2 };

// Store one quantized-then-dequantized activation (element k of batch row m) into its panel.
__device__ __forceinline__ void panel_store(uint8_t *__restrict__ Xp, int kind, int m, int k, float xhat, float gsum) {
    if (kind == RD_PANEL_Q4K) {
        half_t *base = (half_t *)(Xp + (size_t)(k >> 8) * RD_Q4K_PANEL_BYTES);
        int t = k & 255, j = t >> 5;
        base[q4k_panel_index(t, m)] = (half_t)xhat;
        if ((t & 31) == 0) base[q4k_panel_sum_index(j, m)] = (half_t)gsum;
        if ((t & 31) == 1) base[q4k_panel_sum_index(j, m) - (j & 3) + 4 + (j & 3)] = (half_t)0.f;
    } else {
        half_t *base = (half_t *)(Xp + (size_t)(k >> 7) * RD_LIN_PANEL_BYTES);
        base[kind == RD_PANEL_LIN ? lin_panel_index(k & 127, m) : lin4_panel_index(k & 127, m)] = (half_t)xhat;
    }
}

// x f32 [M][K] -> panels. Grid (K/256, M), 256 threads: thread t is element t of the 256-wide chunk.
extern "C" __global__ __launch_bounds__(256) void rd_k_quant_act(const float *__restrict__ x, uint8_t *__restrict__ Xp, int K, int kind) {
    int m = blockIdx.y, k = blockIdx.x * 256 + threadIdx.x;
    float v = k < K ? x[(size_t)m * K + k] : 0.f;
    float gs, xh = quant_g32(v, &gs);
    if (k < K) panel_store(Xp, kind, m, k, xh, gs);
}

// out[m][n] = sum_s P[s][m][n] in ascending split order (deterministic).
extern "C" __global__ void rd_k_reduce_splits(const float *__restrict__ P, float *__restrict__ out, int N, int splits) {
    int m = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x;
    if (n >= N) return;
    float a = P[(size_t)m * N + n];
    for (int s = 1; s < splits; s++) a = __fadd_rn(a, P[((size_t)s * 32 + m) * N + n]);
    out[(size_t)m * N + n] = a;
}

// One block per batch row:  h[m] (+)= sum_s P[s][m][:]   (residual add of a split-K GEMM result, when P != nullptr)
//                           normed = (h*inv)*w with inv = f32(1/sqrt(ss/H+eps)), ss summed in f64   (decoder/rmsnorm.go:29-92)
//                           panels <- per-32 quantization of normed                                  (weightmat.go:33-38)
// Optionally writes normed f32 to norm_out (used by MoE routing, which reads the un-quantized row).
extern "C" __global__ __launch_bounds__(256) void rd_k_add_rmsnorm_quant(float *__restrict__ h, const float *__restrict__ P, int splits,
                                                                         const float *__restrict__ w, float eps, int H,
                                                                         uint8_t *__restrict__ Xp, int kind, float *__restrict__ norm_out) {
    __shared__ double red[4];
    int m = blockIdx.x, t = threadIdx.x;
    float *hr = h + (size_t)m * H;
    float vals[32]; // H <= 8192
    double ss = 0;
#pragma unroll
    for (int i = 0; i < 32; i++) {
        int k = t + i * 256;
        if (k < H) {
            float v = hr[k];
            if (P) {
                float a = P[(size_t)m * H + k];
                for (int s = 1; s < splits; s++) a = __fadd_rn(a, P[((size_t)s * 32 + m) * H + k]);
                v = __fadd_rn(v, a);
                hr[k] = v;
            }
            vals[i] = v;
            ss += (double)v * (double)v;
        }
    }
    ss = wave_sum64_d(ss);
    if ((t & 63) == 0) red[t >> 6] = ss;
    __syncthreads();
    ss = (red[0] + red[1]) + (red[2] + red[3]);
    float inv = (float)(1.0 / sqrt(ss / (double)H + (double)eps));
#pragma unroll
    for (int i = 0; i < 32; i++) {
        int k = t + i * 256;
        if (k < H) {
            float nv = __fmul_rn(__fmul_rn(vals[i], inv), w[k]);
            if (norm_out) norm_out[(size_t)m * H + k] = nv;
            float gs, xh = quant_g32(nv, &gs);
            panel_store(Xp, kind, m, k, xh, gs);
        }
    }
}

// gate/up partials P[s][32][2I] -> act = silu(gate)*up (decoder/rmsnorm.go:204-207: silu in f64) -> per-32 quant -> panels.
// Grid (ceil(I/256), M).
extern "C" __global__ __launch_bounds__(256) void rd_k_swiglu_quant(const float *__restrict__ P, int splits, int I, uint8_t *__restrict__ Xp,
                                                                    int kind, float *__restrict__ act_out) {
    int m = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x;
    float a = 0.f;
    if (n < I) {
        int N2 = 2 * I;
        float g = P[(size_t)m * N2 + n], u = P[(size_t)m * N2 + I + n];
        for (int s = 1; s < splits; s++) {
            g = __fadd_rn(g, P[((size_t)s * 32 + m) * N2 + n]);
            u = __fadd_rn(u, P[((size_t)s * 32 + m) * N2 + I + n]);
        }
        double g64 = (double)g;
        float sl = (float)(g64 / (1.0 + exp(-g64)));
        a = __fmul_rn(sl, u);
        if (act_out) act_out[(size_t)m * I + n] = a;
    }
    float gs, xh = quant_g32(a, &gs);
    if (n < I) panel_store(Xp, kind, m, n, xh, gs);
}
