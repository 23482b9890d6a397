/*
 * oracle.c — CPU restatement of goinfer's ragged batched decode step. TEST INFRASTRUCTURE ONLY:
 * see oracle.h for the contract, the reference citations and the pin status of every function.
 * Build with -ffp-contract=off: the Go reference rounds every f32 operation (amd64 never fuses).
 */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 1;
void or_set_threads(int n) { g_threads = n < 1 ? 1 : n; }

/* A deliberately WRONG oracle, for one purpose: to measure how large a mistake each parity test would catch
 * (tests/test_oracle_mutants.py). 0 = the faithful restatement (the default and the only value any parity check runs with). */
static int g_fault = 0;
void or_set_fault(int f) { g_fault = f; }

/* ------------------------------------------------------------------ f16 */
/* internal/runtime/f16/f16.go:14-43 (Bits): round-half-up on the dropped mantissa bits. */
uint16_t or_f32_to_f16(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    uint16_t sign = (uint16_t)((b >> 16) & 0x8000);
    int32_t e = (int32_t)((b >> 23) & 0xFF) - 112;
    uint32_t m = b & 0x7FFFFF;
    if (((b >> 23) & 0xFF) == 0xFF) return m ? (sign | 0x7E00) : (sign | 0x7C00);
    if (e >= 0x1F) return sign | 0x7C00;
    if (e <= 0) {
        if (e < -10) return sign;
        m |= 0x800000;
        uint32_t sh = (uint32_t)(14 - e);
        return sign | (uint16_t)((m + (1u << (sh - 1))) >> sh);
    }
    uint16_t half = sign | (uint16_t)(e << 10) | (uint16_t)(m >> 13);
    if (m & 0x1000) half++;
    return half;
}

/* internal/runtime/f16/f16.go:46-63 (ToF32): exact widening. */
float or_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000) << 16;
    uint32_t exp = (h >> 10) & 0x1F, man = h & 0x3FF, u;
    float f;
    if (exp == 0) {
        if (man == 0) {
            u = sign;
            memcpy(&f, &u, 4);
            return f;
        }
        f = (float)man / 1024.0f * 6.103515625e-05f; /* 2^-14 */
        return sign ? -f : f;
    }
    if (exp == 0x1F)
        u = sign | 0x7F800000u | (man << 13);
    else
        u = sign | ((exp + 112) << 23) | (man << 13);
    memcpy(&f, &u, 4);
    return f;
}

/* ------------------------------------------------------------------ Q4_K */
/* ggml get_scale_min_k4: backend/cuda/actgroup.cu:64-75, backend/metal/kernels/gemm_kq_test.go:31-36. */
void or_q4k_scale_min(int j, const uint8_t *q, int *sc, int *m) {
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (q[j + 4] & 15) | ((q[j - 4] >> 6) << 4);
        *m = (q[j + 4] >> 4) | ((q[j] >> 6) << 4);
    }
}

/* decoder/gguf.go:1508-1537 (q4kMat wraps the raw blocks) and gemm_kq_test.go:58-68: element e of a
 * block, j=e/32, l=e%32, q=(qs[(j/2)*32+l]>>(4*(j&1)))&15, w = d*sc_j*q - dmin*m_j in f32 with the
 * two products (d*sc), (dmin*m) formed first. */
void or_dequant_q4k(const uint8_t *blocks, size_t n_blocks, float *out) {
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * 144;
        float d = or_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        float dmin = or_f16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
        const uint8_t *qs = blk + 16;
        float *o = out + b * 256;
        for (int j = 0; j < 8; j++) {
            int sc, m;
            or_q4k_scale_min(j, blk + 4, &sc, &m);
            float d1 = d * (float)sc, m1 = dmin * (float)m;
            for (int l = 0; l < 32; l++) {
                int q = (qs[(j / 2) * 32 + l] >> (4 * (j & 1))) & 15;
                o[j * 32 + l] = d1 * (float)q - m1;
            }
        }
    }
}

/* The public ggml Q5_K layout (ggml-quants dequantize_row_q5_K; the reference's kernels state it at
 * backend/cuda/actgroup.cu:77-137): 64 elements per pass, low nibbles then high nibbles of qs[32*pass..], fifth bits from
 * bits 2*pass and 2*pass+1 of qh[l]. Products d*sc and dmin*m formed first, as for Q4_K. */
static inline int q5k_code(const uint8_t *blk, int e) {
    int j = e / 32, l = e % 32;
    int nib = (blk[48 + (j / 2) * 32 + l] >> (4 * (j & 1))) & 15;
    return nib | (((blk[16 + l] >> j) & 1) << 4);
}
void or_dequant_q5k(const uint8_t *blocks, size_t n_blocks, float *out) {
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * 176;
        float d = or_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        float dmin = or_f16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
        float *o = out + b * 256;
        for (int j = 0; j < 8; j++) {
            int sc, m;
            or_q4k_scale_min(j, blk + 4, &sc, &m);
            float d1 = d * (float)sc, m1 = dmin * (float)m;
            for (int l = 0; l < 32; l++) o[j * 32 + l] = d1 * (float)q5k_code(blk, j * 32 + l) - m1;
        }
    }
}

/* The public ggml Q6_K layout (dequantize_row_q6_K; backend/cuda/actgroup.cu:139-205): two halves of 128 elements; in a
 * half, element 32*g + l (g = 0..3) takes its nibble from ql[64*half + 32*(g&1) + l] (low for g < 2, high above) and its two
 * high bits from bits 2g, 2g+1 of qh[32*half + l]; its sub-block scale is sc[8*half + 2*g + l/16]. w = (d*sc) * (q-32). */
static inline int q6k_code(const uint8_t *blk, int e) {
    int half = e / 128, r = e % 128, g = r / 32, l = r % 32;
    int nib = (blk[64 * half + 32 * (g & 1) + l] >> (4 * (g >> 1))) & 15;
    int hi = (blk[128 + 32 * half + l] >> (2 * g)) & 3;
    return (nib | (hi << 4)) - 32;
}
static inline int q6k_scale(const uint8_t *blk, int e) {
    int half = e / 128, r = e % 128, g = r / 32, l = r % 32;
    return (int)(int8_t)blk[192 + 8 * half + 2 * g + l / 16];
}
void or_dequant_q6k(const uint8_t *blocks, size_t n_blocks, float *out) {
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * 210;
        float d = or_f16_to_f32((uint16_t)(blk[208] | (blk[209] << 8)));
        float *o = out + b * 256;
        for (int e = 0; e < 256; e++) o[e] = (d * (float)q6k_scale(blk, e)) * (float)q6k_code(blk, e);
    }
}

/* ------------------------------------------------------------------ int8 rows back to f32 */
/* decoder/kvcache.go:54-59 (dequantHeads -> linalg.DequantizeRowsInt8Into), backend/cuda/kvtype.cuh:48-52 (KV_LDS):
 * dst[r][c] = (float)q[r][c] * scales[r], one f32 product per element. */
void or_dequantize_rows_int8(float *dst, const int8_t *q, const float *scales, int rows, int cols) {
    for (int r = 0; r < rows; r++)
        for (int c = 0; c < cols; c++) dst[(size_t)r * cols + c] = (float)q[(size_t)r * cols + c] * scales[r];
}

/* ------------------------------------------------------------------ activation quantizers */
static inline float round_half_away(float x) { return roundf(x); }

/* backend/cuda/kv8_store.cu:3-5,27-35 (states aikit linalg.QuantizeRowInt8): scale = maxabs/127 in f32,
 * q = round-half-away(x * (1/scale)) clamped to [-127,127]; an all-zero row gets scale 1 and zeros. */
float or_quantize_row_int8(const float *row, int n, int8_t *q) {
    float ma = 0.f;
    for (int i = 0; i < n; i++) {
        float a = fabsf(row[i]);
        if (a > ma) ma = a;
    }
    if (ma == 0.f) {
        memset(q, 0, (size_t)n);
        return 1.f;
    }
    float sc = ma / 127.f, inv = 1.f / sc;
    for (int i = 0; i < n; i++) {
        float x = round_half_away(row[i] * inv);
        if (x > 127.f) x = 127.f;
        if (x < -127.f) x = -127.f;
        q[i] = (int8_t)(int)x;
    }
    return sc;
}

/* aikit linalg.QuantizeActQ as called at decoder/cpu_gateup_fused.go:110-117 and weightmat.go:845-862:
 * group 0 = QuantizeRowInt8 per row; group g = the same rule over every g consecutive elements
 * (a ragged last group included), in-tree twin backend/cuda/actgroup.cu:32-54. */
void or_quantize_act(const float *a, int M, int K, int group, int8_t *q, float *S) {
    if (group <= 0) {
        for (int m = 0; m < M; m++) S[m] = or_quantize_row_int8(a + (size_t)m * K, K, q + (size_t)m * K);
        return;
    }
    int nG = (K + group - 1) / group;
    for (int m = 0; m < M; m++)
        for (int g = 0; g < nG; g++) {
            int lo = g * group, n = K - lo < group ? K - lo : group;
            S[(size_t)m * nG + g] = or_quantize_row_int8(a + (size_t)m * K + lo, n, q + (size_t)m * K + lo);
        }
}

/* ------------------------------------------------------------------ int4 g32 */
/* decoder/fakequant.go:52-56,99-131 ("sym", aikit's runtime int4): scale = maxabs/group... /7, zero group -> 1,
 * code = clamp(round-half-away(v/s), -7, 7); canonical packing backend/cuda/internal/wpack/wpack.go:165-207
 * and kernels/actgroup_kernel_test.go:252-261: element k in nibble k%2 (low first) of byte k/2, stored nib = code+8. */
void or_quantize_int4_row(const float *row, int cols, int group, uint8_t *packed, float *scales) {
    memset(packed, 0, (size_t)((cols + 1) / 2));
    int nG = (cols + group - 1) / group;
    for (int g = 0; g < nG; g++) {
        int lo = g * group, hi = lo + group < cols ? lo + group : cols;
        float mx = 0.f;
        for (int k = lo; k < hi; k++) {
            float a = fabsf(row[k]);
            if (a > mx) mx = a;
        }
        float s = mx > 0.f ? mx / 7.f : 1.f;
        float inv = 1.f / s;
        scales[g] = s;
        for (int k = lo; k < hi; k++) {
            float c = round_half_away(row[k] * inv);
            if (c > 7.f) c = 7.f;
            if (c < -7.f) c = -7.f;
            uint8_t nib = (uint8_t)((int)c + 8);
            packed[k >> 1] |= (uint8_t)(nib << (4 * (k & 1)));
        }
    }
}

/* decoder/weightmat.go:166-178 (streamQuantizedRow4, quantInt4): per row QuantizeGroupInt4Row then the
 * f32 group scales narrowed to binary16. */
void or_quantize_int4_mat(const float *w, int rows, int cols, int group, uint8_t *q4, uint16_t *s16) {
    int nG = (cols + group - 1) / group, bpr = (cols + 1) / 2;
    float *sc = (float *)malloc(sizeof(float) * (size_t)nG);
    for (int r = 0; r < rows; r++) {
        or_quantize_int4_row(w + (size_t)r * cols, cols, group, q4 + (size_t)r * bpr, sc);
        for (int g = 0; g < nG; g++) s16[(size_t)r * nG + g] = or_f32_to_f16(sc[g]);
    }
    free(sc);
}

/* ------------------------------------------------------------------ attention primitives */
/* aikit linalg.MatmulQKAcc64 as called at decoder/forwardn.go:379-383: dst[i,s] = f32(sum_d f64(a[i,d])*f64(k[s,off+d])),
 * d ascending (decoder/attention.go:335-352 dotsF64x8 states the same fold). */
void or_qk_acc64(const float *a, const float *keys, float *dst, int M, int hd, int nKeys, int off, int kvDim) {
    for (int i = 0; i < M; i++)
        for (int s = 0; s < nKeys; s++) {
            const float *k = keys + (size_t)s * kvDim + off;
            double acc = 0;
            for (int d = 0; d < hd; d++) acc += (double)a[i * hd + d] * (double)k[d];
            dst[(size_t)i * nKeys + s] = (float)acc;
        }
}

/* aikit linalg.MatmulAVAcc64 as called at decoder/forwardn.go:488-490: hd independent f64 accumulators,
 * key-ascending adds, rounded to f32 once. */
void or_av_acc64(const float *scores, const float *vals, float *dst, int M, int nKeys, int hd, int off, int kvDim) {
    double *acc = (double *)malloc(sizeof(double) * (size_t)hd);
    for (int i = 0; i < M; i++) {
        for (int d = 0; d < hd; d++) acc[d] = 0;
        for (int s = 0; s < nKeys; s++) {
            double w = (double)scores[(size_t)i * nKeys + s];
            const float *v = vals + (size_t)s * kvDim + off;
            for (int d = 0; d < hd; d++) acc[d] += w * (double)v[d];
        }
        for (int d = 0; d < hd; d++) dst[i * hd + d] = (float)acc[d];
    }
    free(acc);
}

/* ------------------------------------------------------------------ glue */
/* decoder/rmsnorm.go:29-92 (rmsNormInto): four f64 partial sums, (ss0+ss1)+(ss2+ss3)+tail. */
void or_rmsnorm(float *dst, const float *src, const float *w, int rows, int dim, double eps, int add_one) {
    for (int r = 0; r < rows; r++) {
        const float *s = src + (size_t)r * dim;
        float *o = dst + (size_t)r * dim;
        double ss0 = 0, ss1 = 0, ss2 = 0, ss3 = 0, tail = 0;
        int i = 0;
        for (; i + 3 < dim; i += 4) {
            double v0 = s[i], v1 = s[i + 1], v2 = s[i + 2], v3 = s[i + 3];
            ss0 += v0 * v0;
            ss1 += v1 * v1;
            ss2 += v2 * v2;
            ss3 += v3 * v3;
        }
        for (; i < dim; i++) tail += (double)s[i] * (double)s[i];
        double ss = (ss0 + ss1) + (ss2 + ss3) + tail;
        float inv = (float)(1.0 / sqrt(ss / (double)dim + eps));
        for (i = 0; i < dim; i++) o[i] = add_one ? (s[i] * inv) * (1.f + w[i]) : (s[i] * inv) * w[i];
    }
}

/* decoder/rope.go:28-64 (applyRoPE, NeoX rotate-half): theta, cos, sin and the rotation in f64. */
void or_rope(float *vec, int heads, int head_dim, int pos, const double *inv_freq, int half, double scale) {
    if (half == 0 || heads == 0) return;
    double c[512], s[512];
    for (int d = 0; d < half; d++) {
        double theta = (double)pos * inv_freq[d];
        c[d] = cos(theta) * scale;
        s[d] = sin(theta) * scale;
    }
    for (int h = 0; h < heads; h++) {
        float *v1 = vec + (size_t)h * head_dim, *v2 = v1 + half;
        for (int d = 0; d < half; d++) {
            double x1 = v1[d], x2 = v2[d];
            v1[d] = (float)(x1 * c[d] - x2 * s[d]);
            v2[d] = (float)(x2 * c[d] + x1 * s[d]);
        }
    }
}

/* decoder/rmsnorm.go:204-207 */
float or_silu(float x) {
    double x64 = x;
    return (float)(x64 / (1 + exp(-x64)));
}

/* decoder/mlp.go:269-290 */
void or_swiglu(float *gate, const float *up, int n) {
    for (int i = 0; i < n; i++) gate[i] = or_silu(gate[i]) * up[i];
}

/* decoder/rmsnorm.go:229-234 (geluTanh): 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) in f64, narrowed once. */
float or_gelu_tanh(float x) {
    const double c = 0.7978845608028654;
    double x64 = x;
    double inner = c * (x64 + 0.044715 * x64 * x64 * x64);
    return (float)(0.5 * x64 * (1 + tanh(inner)));
}

void or_geglu(float *gate, const float *up, int n) {
    for (int i = 0; i < n; i++) gate[i] = or_gelu_tanh(gate[i]) * up[i];
}

/* decoder/model_forward.go:259-266 (softcapParallel): the division in f32, tanh in f64, the product in f32. */
void or_softcap_logits(float *logits, size_t n, float cap) {
    for (size_t i = 0; i < n; i++) logits[i] = cap * (float)tanh((double)(logits[i] / cap));
}

/* decoder/mlp.go:370-410 (softmaxF32): f32 max, e=exp(f64(x-max)) stored f32, f64 sum, out*=f32(1/sum). */
void or_softmax_f32(const float *x, int n, float *out) {
    if (n == 0) return;
    float mx = x[0];
    for (int i = 1; i < n; i++)
        if (x[i] > mx) mx = x[i];
    double sum = 0;
    for (int i = 0; i < n; i++) {
        double e = exp((double)(x[i] - mx));
        out[i] = (float)e;
        sum += e;
    }
    float inv = (float)(1.0 / sum);
    for (int i = 0; i < n; i++) out[i] *= inv;
}

/* decoder/mlp.go:414-440 (topK): k passes of strict '>' — the lowest index wins a tie. */
int or_topk(const float *x, int n, int k, int *idx, float *val) {
    unsigned char *used = (unsigned char *)calloc((size_t)n, 1);
    int cnt = 0;
    for (; k > 0; k--) {
        float best = -INFINITY;
        int bi = -1;
        for (int i = 0; i < n; i++)
            if (!used[i] && x[i] > best) {
                best = x[i];
                bi = i;
            }
        if (bi < 0) break;
        used[bi] = 1;
        idx[cnt] = bi;
        if (val) val[cnt] = best;
        cnt++;
    }
    free(used);
    return cnt;
}

/* decoder/mlp.go:186-228 (groupLimit): DeepSeek-V3 group-limited selection. The nE selection scores fall into nGroup contiguous
 * groups of nE/nGroup; a group's score is the sum of its two largest entries; the topkGroup best groups (topK's rule) keep their
 * scores, everything else, the experts past nGroup*(nE/nGroup) included, becomes -inf. out may not alias sel. */
void or_group_limit(const float *sel, int nE, int nGroup, int topkGroup, float *out) {
    int gsz = nE / nGroup;
    float *gscore = (float *)malloc(sizeof(float) * (size_t)nGroup);
    int *keepIdx = (int *)malloc(sizeof(int) * (size_t)(topkGroup > 0 ? topkGroup : 1));
    for (int g = 0; g < nGroup; g++) {
        float top1 = -INFINITY, top2 = -INFINITY;
        for (int i = g * gsz; i < (g + 1) * gsz; i++) {
            float v = sel[i];
            if (v > top1) {
                top2 = top1;
                top1 = v;
            } else if (v > top2) {
                top2 = v;
            }
        }
        gscore[g] = top1 + top2;
    }
    int nk = or_topk(gscore, nGroup, topkGroup, keepIdx, NULL);
    for (int i = 0; i < nE; i++) out[i] = -INFINITY;
    for (int j = 0; j < nk; j++)
        for (int i = keepIdx[j] * gsz; i < (keepIdx[j] + 1) * gsz; i++) out[i] = sel[i];
    free(gscore);
    free(keepIdx);
}

/* decoder/mlp.go:130-184 (routeExperts). Scores: softmax over the experts, or (sigmoid) each expert's own
 * float32(1/(1+exp(-float64(logit)))). Selection scores: scores + bias when there is a bias (e_score_correction_bias), masked by
 * or_group_limit when nGroup > 1; the k best by topK's rule. Weights: the chosen experts' UNBIASED scores; norm divides them by
 * their f32 sum taken in rank order (when it is > 0); scale multiplies them when it is neither 0 nor 1. */
int or_route_experts_ex(const float *logits, const float *bias, int nE, int k, int sigmoid, int norm, double scale, int nGroup,
                        int topkGroup, int *idx, float *wts) {
    float *scores = (float *)malloc(sizeof(float) * (size_t)nE), *sel = scores, *lim = NULL;
    if (sigmoid)
        for (int i = 0; i < nE; i++) scores[i] = (float)(1.0 / (1.0 + exp(-(double)logits[i])));
    else
        or_softmax_f32(logits, nE, scores);
    if (bias) {
        sel = (float *)malloc(sizeof(float) * (size_t)nE);
        for (int i = 0; i < nE; i++) sel[i] = scores[i] + bias[i];
    }
    if (nGroup > 1) {
        lim = (float *)malloc(sizeof(float) * (size_t)nE);
        or_group_limit(sel, nE, nGroup, topkGroup, lim);
    }
    int n = or_topk(lim ? lim : sel, nE, k, idx, NULL);
    for (int j = 0; j < n; j++) wts[j] = scores[idx[j]];
    if (norm) {
        float s = 0.f;
        for (int j = 0; j < n; j++) s += wts[j];
        if (s > 0.f)
            for (int j = 0; j < n; j++) wts[j] /= s;
    }
    if (scale != 0 && scale != 1)
        for (int j = 0; j < n; j++) wts[j] *= (float)scale;
    if (sel != scores) free(sel);
    free(lim);
    free(scores);
    return n;
}
int or_route_experts(const float *logits, int nE, int k, int norm, double scale, int *idx, float *wts) {
    return or_route_experts_ex(logits, NULL, nE, k, 0, norm, scale, 0, 0, idx, wts);
}

/* internal/runtime/sampling/sampler.go:485-520 (Argmax): strict '>' from index 0. */
int or_argmax(const float *x, int n) {
    int bi = 0;
    float best = x[0];
    for (int i = 1; i < n; i++)
        if (x[i] > best) {
            best = x[i];
            bi = i;
        }
    return bi;
}

/* ------------------------------------------------------------------ the K best logits of a row */
/* internal/runtime/sampling/sampler.go:726-782 (topKByLogit): a k-bounded min-heap whose root is the worst kept entry, "worse" being
 * the lower logit or, on a tie, the LARGER id; then the order its callers give the result, (logit descending, id ascending)
 * (sampler_topk.go:10-15, decoder/resident/forward.go:86-90). ids, vals: min(k, n) entries. Returns that count. */
static int topk_worse(const float *x, int a, int b) { return x[a] != x[b] ? x[a] < x[b] : a > b; }
int or_topk_by_logit(const float *x, int n, int k, int *ids, float *vals) {
    if (k > n) k = n;
    if (k <= 0) return 0;
    int *h = (int *)malloc(sizeof(int) * (size_t)k), len = 0;
    for (int id = 0; id < n; id++) {
        if (len < k) {
            int i = len;
            h[len++] = id;
            while (i > 0) { /* siftUp: a child worse than its parent moves toward the root */
                int p = (i - 1) / 2;
                if (!topk_worse(x, h[i], h[p])) break;
                int t = h[p];
                h[p] = h[i], h[i] = t, i = p;
            }
        } else if (topk_worse(x, h[0], id)) { /* the candidate is better than the worst kept */
            h[0] = id;
            for (int i = 0;;) { /* siftDownRoot */
                int l = 2 * i + 1, r = 2 * i + 2, m = i;
                if (l < len && topk_worse(x, h[l], h[m])) m = l;
                if (r < len && topk_worse(x, h[r], h[m])) m = r;
                if (m == i) break;
                int t = h[i];
                h[i] = h[m], h[m] = t, i = m;
            }
        }
    }
    /* (logit desc, id asc): insertion sort, k <= 1024 */
    for (int i = 1; i < len; i++) {
        int v = h[i], j = i - 1;
        while (j >= 0 && topk_worse(x, h[j], v)) h[j + 1] = h[j], j--;
        h[j + 1] = v;
    }
    for (int i = 0; i < len; i++) ids[i] = h[i], vals[i] = x[h[i]];
    free(h);
    return len;
}

/* The top-p denominator as the host forms every probability (sampler.go:784-800 topPCandidates, sampler_chunked.go:136-141 chunkedZ):
 * sum over the row of exp((f64(l) - max) / T), here in plain ascending order (the host's fixed chunking regroups the same f64
 * terms; the difference is a few ulp of f64). */
double or_softmax_z(const float *x, int n, double temperature) {
    double mx = x[0], z = 0;
    for (int i = 1; i < n; i++)
        if (x[i] > mx) mx = x[i];
    for (int i = 0; i < n; i++) z += exp(((double)x[i] - mx) / temperature);
    return z;
}

/* ------------------------------------------------------------------ temperature-only sampling (Gumbel-max) */
/* internal/runtime/sampling/philox.go:13-40 (Philox4x32): Philox4x32-10; the key is bumped between rounds, not before the first. */
void or_philox4x32(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; r++) {
        if (r > 0) k0 += 0x9E3779B9u, k1 += 0xBB67AE85u;
        uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        c0 = n0, c1 = (uint32_t)p1, c2 = n2, c3 = (uint32_t)p0;
    }
    out[0] = c0, out[1] = c1, out[2] = c2, out[3] = c3;
}

/* sampler_gumbel.go:33-37 (gumbelNoise): w = (h + 0.5) / 2^32 in f64, E = -log1p(-w), G = f32(-log(E)). */
float or_gumbel_noise(uint32_t h) {
    double w = ((double)h + 0.5) * (1.0 / 4294967296.0);
    double e = -log1p(-w);
    return (float)(-log(e));
}

/* sampler_gumbel.go:41-43 (GumbelKey): the product is rounded to f32 before the add (no fused multiply-add). */
float or_gumbel_key(float logit, float invT, uint32_t h) {
    volatile float prod = logit * invT;
    return prod + or_gumbel_noise(h);
}

/* sampler_gumbel.go:47-66 (GumbelArgmaxRange over the whole row) and :117-123 (GumbelDraw): counter (i>>2, draw, draw>>32, 0),
 * key (seed, seed>>32), lane i&3; strict '>' from -Inf in ascending index order, so the lowest index wins a tie and a NaN or
 * -Inf key is never chosen; no comparable entry -> the plain argmax. */
int or_gumbel_draw(const float *logits, int n, double temperature, uint64_t seed, uint64_t draw) {
    float invT = (float)(1.0 / temperature);
    uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    float best = -INFINITY;
    int idx = -1;
    for (int b = 0; (b << 2) < n; b++) {
        uint32_t ctr[4] = {(uint32_t)b, (uint32_t)draw, (uint32_t)(draw >> 32), 0}, r[4];
        or_philox4x32(ctr, key, r);
        for (int lane = 0; lane < 4; lane++) {
            int i = (b << 2) + lane;
            if (i >= n) continue;
            float k = or_gumbel_key(logits[i], invT, r[lane]);
            if (k > best) best = k, idx = i;
        }
    }
    return idx < 0 ? or_argmax(logits, n) : idx;
}

/* sampler_gumbel.go:79-109 (Sampler.gumbelDraw): the guards in front of the draw — a temperature <= 0 means 1, and a
 * temperature so small that 1/T overflows f32 is the argmax, as greedy. */
int or_sampler_gumbel_draw(const float *logits, int n, double temperature, uint64_t seed, uint64_t draw) {
    if (temperature <= 0) temperature = 1;
    float invT = (float)(1.0 / temperature);
    if (isinf(invT)) return or_argmax(logits, n);
    return or_gumbel_draw(logits, n, temperature, seed, draw);
}

/* Test conveniences: `count` consecutive draws of one row (draw0, draw0+1, ...), and the noise of many words. */
void or_gumbel_draw_many(const float *logits, int n, double temperature, uint64_t seed, uint64_t draw0, int count, int *out) {
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int i = 0; i < count; i++) out[i] = or_gumbel_draw(logits, n, temperature, seed, draw0 + (uint64_t)i);
}
void or_gumbel_noise_many(const uint32_t *h, size_t n, float *out) {
    for (size_t i = 0; i < n; i++) out[i] = or_gumbel_noise(h[i]);
}

/* ------------------------------------------------------------------ matmul dispatch */
/* decoder/weightmat.go:892-985 (matmulWS): the weight's kind picks the kernel. The int kinds quantize
 * the activation first (group 32 in q4k mode, weightmat.go:33-38). Arithmetic of each row:
 *   q4k   backend/cuda/actgroup.cu:298-355  facc += idot_g*((d*sc_g)*aS_g); facc += -(dmin*m_g)*asum_g
 *   w4a8  backend/cuda/actgroup.cu:243-275  facc += idot_g*(f16(ws_g)*aS_g)      (per-row acts: *aS once at the end)
 *   w8a8  backend/cuda/actgroup.cu:283-288,421-437  facc += idot_g*aS_g; dst = facc*wScale[n]
 * groups ascending, one f32 accumulator per output. */
static void matmul_q4k(const or_mat *w, const int8_t *aq, const float *aS, int M, float *dst) {
    int N = w->N, K = w->K, nSB = K / 256, nG = K / 32;
    const uint8_t *W = (const uint8_t *)w->data;
    float *asum = (float *)malloc(sizeof(float) * (size_t)M * nG);
    for (int m = 0; m < M; m++)
        for (int g = 0; g < nG; g++) {
            int s = 0;
            for (int i = 0; i < 32; i++) s += aq[(size_t)m * K + g * 32 + i];
            asum[(size_t)m * nG + g] = aS[(size_t)m * nG + g] * (float)s;
        }
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int n = 0; n < N; n++) {
        const uint8_t *row = W + (size_t)n * nSB * 144;
        uint8_t qb[256];
        for (int m = 0; m < M; m++) dst[(size_t)m * N + n] = 0.f;
        for (int b = 0; b < nSB; b++) {
            const uint8_t *blk = row + (size_t)b * 144;
            float d = or_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
            float dmin = or_f16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
            int sc[8], mn[8];
            for (int j = 0; j < 8; j++) or_q4k_scale_min(j, blk + 4, &sc[j], &mn[j]);
            for (int p = 0; p < 4; p++)
                for (int l = 0; l < 32; l++) {
                    uint8_t by = blk[16 + p * 32 + l];
                    qb[(2 * p) * 32 + l] = by & 15;
                    qb[(2 * p + 1) * 32 + l] = by >> 4;
                }
            for (int m = 0; m < M; m++) {
                const int8_t *a = aq + (size_t)m * K + b * 256;
                float facc = dst[(size_t)m * N + n];
                for (int j = 0; j < 8; j++) {
                    int32_t idot = 0;
                    for (int l = 0; l < 32; l++) idot += (int32_t)qb[j * 32 + l] * (int32_t)a[j * 32 + l];
                    int g = b * 8 + j;
                    const int js = g_fault == OR_FAULT_Q4K_SCALE_INDEX ? (j + 1) & 7 : j; /* fault: the neighbouring sub-block's scale */
                    facc = fmaf((float)idot, (d * (float)sc[js]) * aS[(size_t)m * nG + g], facc);
                    if (g_fault != OR_FAULT_Q4K_NO_MIN) facc = fmaf(-(dmin * (float)mn[j]), asum[(size_t)m * nG + g], facc);
                }
                dst[(size_t)m * N + n] = facc;
            }
        }
    }
    free(asum);
}

/* Q5_K x per-32 int8 activations, backend/cuda/actgroup.cu:85-137 (rowsQ5K): per 32-group
 * facc = fma(idot, (d*sc)*aS, facc); facc = fma(-(dmin*m), asum, facc), groups ascending. */
static void matmul_q5k(const or_mat *w, const int8_t *aq, const float *aS, int M, float *dst) {
    int N = w->N, K = w->K, nSB = K / 256, nG = K / 32;
    const uint8_t *W = (const uint8_t *)w->data;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int n = 0; n < N; n++) {
        const uint8_t *row = W + (size_t)n * nSB * 176;
        for (int m = 0; m < M; m++) {
            const int8_t *a = aq + (size_t)m * K;
            float facc = 0.f;
            for (int b = 0; b < nSB; b++) {
                const uint8_t *blk = row + (size_t)b * 176;
                float d = or_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
                float dmin = or_f16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
                for (int j = 0; j < 8; j++) {
                    int sc, mn;
                    or_q4k_scale_min(j, blk + 4, &sc, &mn);
                    int32_t idot = 0, asum = 0;
                    for (int l = 0; l < 32; l++) {
                        idot += (int32_t)q5k_code(blk, j * 32 + l) * (int32_t)a[b * 256 + j * 32 + l];
                        asum += a[b * 256 + j * 32 + l];
                    }
                    int g = b * 8 + j;
                    float as = aS[(size_t)m * nG + g];
                    facc = fmaf((float)idot, (d * (float)sc) * as, facc);
                    facc = fmaf(-(dmin * (float)mn), as * (float)asum, facc);
                }
            }
            dst[(size_t)m * N + n] = facc;
        }
    }
}

/* Q6_K x per-32 int8 activations, backend/cuda/actgroup.cu:139-205 (rowsQ6K): an activation group of 32 spans two 16-element
 * sub-blocks; facc = fma((float)(sc_lo*idot_lo + sc_hi*idot_hi), d*aS, facc) in the mathematically specified form (the CUDA
 * lanes fold sc*idot per 8 elements; the integer part is exact either way), groups ascending. */
static void matmul_q6k(const or_mat *w, const int8_t *aq, const float *aS, int M, float *dst) {
    int N = w->N, K = w->K, nSB = K / 256, nG = K / 32;
    const uint8_t *W = (const uint8_t *)w->data;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int n = 0; n < N; n++) {
        const uint8_t *row = W + (size_t)n * nSB * 210;
        for (int m = 0; m < M; m++) {
            const int8_t *a = aq + (size_t)m * K;
            float facc = 0.f;
            for (int b = 0; b < nSB; b++) {
                const uint8_t *blk = row + (size_t)b * 210;
                float d = or_f16_to_f32((uint16_t)(blk[208] | (blk[209] << 8)));
                for (int j = 0; j < 8; j++) {
                    int32_t acc = 0;
                    for (int h = 0; h < 2; h++) {
                        int32_t idot = 0;
                        for (int l = 0; l < 16; l++) {
                            int e = j * 32 + h * 16 + l;
                            idot += (int32_t)q6k_code(blk, e) * (int32_t)a[b * 256 + e];
                        }
                        acc += (int32_t)q6k_scale(blk, j * 32 + h * 16) * idot;
                    }
                    facc = fmaf((float)acc, d * aS[(size_t)m * nG + b * 8 + j], facc);
                }
            }
            dst[(size_t)m * N + n] = facc;
        }
    }
}

static void matmul_w4a8(const or_mat *w, const int8_t *aq, const float *aS, int M, float *dst) {
    int N = w->N, K = w->K, nG = (K + 31) / 32, bpr = (K + 1) / 2, ag = w->act_group;
    const uint8_t *W = (const uint8_t *)w->data;
    const uint16_t *S16 = (const uint16_t *)w->scales;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int n = 0; n < N; n++) {
        const uint8_t *row = W + (size_t)n * bpr;
        for (int m = 0; m < M; m++) {
            const int8_t *a = aq + (size_t)m * K;
            float facc = 0.f;
            for (int g = 0; g < nG; g++) {
                int lo = g * 32, hi = lo + 32 < K ? lo + 32 : K;
                int32_t idot = 0;
                for (int k = lo; k < hi; k++) {
                    int c = (int)((row[k >> 1] >> (4 * (k & 1))) & 15) - 8;
                    idot += c * (int32_t)a[k];
                }
                float ws = or_f16_to_f32(S16[(size_t)n * nG + (g_fault == OR_FAULT_W4A8_SCALE_INDEX ? (g + 1) % nG : g)]);
                if (ag > 0)
                    facc = fmaf((float)idot, ws * aS[(size_t)m * nG + g], facc);
                else
                    facc = fmaf((float)idot, ws, facc);
            }
            dst[(size_t)m * N + n] = ag > 0 ? facc : facc * aS[m];
        }
    }
}

static void matmul_w8a8(const or_mat *w, const int8_t *aq, const float *aS, int M, float *dst) {
    int N = w->N, K = w->K, nG = (K + 31) / 32, ag = w->act_group;
    const int8_t *W = (const int8_t *)w->data;
    const float *wS = (const float *)w->scales;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int n = 0; n < N; n++) {
        const int8_t *row = W + (size_t)n * K;
        for (int m = 0; m < M; m++) {
            const int8_t *a = aq + (size_t)m * K;
            if (ag > 0) {
                float facc = 0.f;
                for (int g = 0; g < nG; g++) {
                    int lo = g * 32, hi = lo + 32 < K ? lo + 32 : K;
                    int32_t idot = 0;
                    for (int k = lo; k < hi; k++) idot += (int32_t)row[k] * (int32_t)a[k];
                    facc = fmaf((float)idot, aS[(size_t)m * nG + g], facc);
                }
                dst[(size_t)m * N + n] = facc * wS[n];
            } else {
                int32_t idot = 0;
                for (int k = 0; k < K; k++) idot += (int32_t)row[k] * (int32_t)a[k];
                dst[(size_t)m * N + n] = ((float)idot * aS[m]) * wS[n];
            }
        }
    }
}

void or_matmul(const or_mat *w, const float *a, int M, float *dst) {
    int N = w->N, K = w->K;
    if (w->kind == OR_F32) {
        const float *W = (const float *)w->data;
#pragma omp parallel for num_threads(g_threads) schedule(static)
        for (int n = 0; n < N; n++)
            for (int m = 0; m < M; m++) {
                double acc = 0;
                for (int k = 0; k < K; k++) acc += (double)a[(size_t)m * K + k] * (double)W[(size_t)n * K + k];
                dst[(size_t)m * N + n] = (float)acc;
            }
        return;
    }
    int group = w->act_group;
    int nG = group > 0 ? (K + group - 1) / group : 1;
    int8_t *aq = (int8_t *)malloc((size_t)M * K);
    float *aS = (float *)malloc(sizeof(float) * (size_t)M * nG);
    or_quantize_act(a, M, K, group, aq, aS);
    if (w->kind == OR_Q4K)
        matmul_q4k(w, aq, aS, M, dst);
    else if (w->kind == OR_Q5K)
        matmul_q5k(w, aq, aS, M, dst);
    else if (w->kind == OR_Q6K)
        matmul_q6k(w, aq, aS, M, dst);
    else if (w->kind == OR_W4A8)
        matmul_w4a8(w, aq, aS, M, dst);
    else
        matmul_w8a8(w, aq, aS, M, dst);
    free(aq);
    free(aS);
}

/* dequantized weight element (n,k) as a double */
static double weight_at(const or_mat *w, int n, int k) {
    switch (w->kind) {
    case OR_F32: return ((const float *)w->data)[(size_t)n * w->K + k];
    case OR_Q4K: {
        const uint8_t *blk = (const uint8_t *)w->data + ((size_t)n * (w->K / 256) + k / 256) * 144;
        int e = k % 256, j = e / 32, l = e % 32, sc, m;
        or_q4k_scale_min(j, blk + 4, &sc, &m);
        double d = or_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        double dmin = or_f16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
        int q = (blk[16 + (j / 2) * 32 + l] >> (4 * (j & 1))) & 15;
        return d * sc * q - dmin * m;
    }
    case OR_Q5K: {
        const uint8_t *blk = (const uint8_t *)w->data + ((size_t)n * (w->K / 256) + k / 256) * 176;
        int e = k % 256, sc, m;
        or_q4k_scale_min(e / 32, blk + 4, &sc, &m);
        double d = or_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
        double dmin = or_f16_to_f32((uint16_t)(blk[2] | (blk[3] << 8)));
        return d * sc * q5k_code(blk, e) - dmin * m;
    }
    case OR_Q6K: {
        const uint8_t *blk = (const uint8_t *)w->data + ((size_t)n * (w->K / 256) + k / 256) * 210;
        int e = k % 256;
        return (double)or_f16_to_f32((uint16_t)(blk[208] | (blk[209] << 8))) * q6k_scale(blk, e) * q6k_code(blk, e);
    }
    case OR_W4A8: {
        int nG = (w->K + 31) / 32, bpr = (w->K + 1) / 2;
        int c = (int)((((const uint8_t *)w->data)[(size_t)n * bpr + (k >> 1)] >> (4 * (k & 1))) & 15) - 8;
        return (double)c * (double)or_f16_to_f32(((const uint16_t *)w->scales)[(size_t)n * nG + k / 32]);
    }
    default: return (double)((const int8_t *)w->data)[(size_t)n * w->K + k] * (double)((const float *)w->scales)[n];
    }
}

void or_matmul_f64ref(const or_mat *w, const float *a, int M, double *dst) {
    int N = w->N, K = w->K;
    double *ad = (double *)malloc(sizeof(double) * (size_t)M * K);
    if (w->kind == OR_F32) {
        for (size_t i = 0; i < (size_t)M * K; i++) ad[i] = a[i];
    } else {
        int group = w->act_group, nG = group > 0 ? (K + group - 1) / group : 1;
        int8_t *aq = (int8_t *)malloc((size_t)M * K);
        float *aS = (float *)malloc(sizeof(float) * (size_t)M * nG);
        or_quantize_act(a, M, K, group, aq, aS);
        for (int m = 0; m < M; m++)
            for (int k = 0; k < K; k++)
                ad[(size_t)m * K + k] = (double)aq[(size_t)m * K + k] * (double)aS[(size_t)m * nG + (group > 0 ? k / group : 0)];
        free(aq);
        free(aS);
    }
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int n = 0; n < N; n++) {
        double *wr = (double *)malloc(sizeof(double) * (size_t)K);
        for (int k = 0; k < K; k++) wr[k] = weight_at(w, n, k);
        for (int m = 0; m < M; m++) {
            double acc = 0;
            for (int k = 0; k < K; k++) acc += ad[(size_t)m * K + k] * wr[k];
            dst[(size_t)m * N + n] = acc;
        }
        free(wr);
    }
    free(ad);
}

/* ------------------------------------------------------------------ attention */
/* decoder/attention.go:287-295 */
static double softcap_score(double s, double c) { return c == 0 ? s : c * tanh(s / c); }

/* decoder/forwardn.go:295-500 with useAcc64 and K=1 (the form program_cpu_n.go:497-515 calls), no sinks,
 * no tree mask: per query head, scores = f32(f64 dot) -> sc = softcap(f64(score)*scale) stored f32 ->
 * max -> e = exp(f64(sc_f32) - max) stored f32, f64 sum -> w = f32(f64(e_f32) * (1/sum)) -> AV in f64. */
void or_attend_sinks(const float *q, float *ctx, const float *keys, const float *vals, int n_keys, int start,
                     int nH, int nKV, int hd, double scale, double softcap, const float *sinks) {
    int kvDim = nKV * hd, group = nH / nKV;
    if (g_fault == OR_FAULT_NO_SOFTCAP) softcap = 0;
#pragma omp parallel for num_threads(g_threads) schedule(dynamic, 1)
    for (int qh = 0; qh < nH; qh++) {
        int kvh = qh / group;
        if (g_fault == OR_FAULT_GQA_HEAD) kvh = (kvh + 1) % nKV; /* fault: the query head reads its neighbour's kv head */
        float *scores = (float *)malloc(sizeof(float) * (size_t)n_keys);
        or_qk_acc64(q + (size_t)qh * hd, keys, scores, 1, hd, n_keys, kvh * hd, kvDim);
        int lo = start < 0 ? 0 : start, hi = n_keys - 1;
        if (g_fault == OR_FAULT_CAUSAL_RANGE && hi > lo) hi--; /* fault: the row does not see its own key */
        if (lo <= hi) {
            double maxS = -INFINITY;
            for (int s = lo; s <= hi; s++) {
                double sc = softcap_score((double)scores[s] * scale, softcap);
                scores[s] = (float)sc;
                if (sc > maxS) maxS = sc;
            }
            /* decoder/attention.go:305-322 sinkMax / sinkSum: the head's learned sink joins the max-shift and the denominator, nothing else */
            if (sinks && (double)sinks[qh] > maxS) maxS = (double)sinks[qh];
            double sum = 0;
            for (int s = lo; s <= hi; s++) {
                double e = exp((double)scores[s] - maxS);
                scores[s] = (float)e;
                sum += e;
            }
            if (sinks) sum += exp((double)sinks[qh] - maxS);
            double inv = 1.0 / sum;
            for (int s = 0; s < lo; s++) scores[s] = 0.f;
            for (int s = lo; s <= hi; s++) scores[s] = (float)((double)scores[s] * inv);
        } else {
            memset(scores, 0, sizeof(float) * (size_t)n_keys);
        }
        or_av_acc64(scores, vals, ctx + (size_t)qh * hd, 1, n_keys, hd, kvh * hd, kvDim);
        free(scores);
    }
}
void or_attend(const float *q, float *ctx, const float *keys, const float *vals, int n_keys, int start,
               int nH, int nKV, int hd, double scale, double softcap) {
    or_attend_sinks(q, ctx, keys, vals, n_keys, start, nH, nKV, hd, scale, softcap, NULL);
}

/* ------------------------------------------------------------------ model */
or_cache *or_cache_new(const or_model *m, int cap) {
    or_cache *c = (or_cache *)calloc(1, sizeof(or_cache));
    size_t kvDim = (size_t)m->n_kv * m->head_dim;
    c->cap = cap;
    c->k = (float **)calloc((size_t)m->n_layers, sizeof(float *));
    c->v = (float **)calloc((size_t)m->n_layers, sizeof(float *));
    for (int l = 0; l < m->n_layers; l++) {
        c->k[l] = (float *)calloc((size_t)cap * kvDim, sizeof(float));
        c->v[l] = (float *)calloc((size_t)cap * kvDim, sizeof(float));
    }
    return c;
}

void or_cache_free(const or_model *m, or_cache *c) {
    if (!c) return;
    for (int l = 0; l < m->n_layers; l++) {
        free(c->k[l]);
        free(c->v[l]);
    }
    free(c->k);
    free(c->v);
    free(c);
}

/* What the cache holds of one position's K or V row [n_kv][hd]: the row itself (f32 cache), its binary16 narrowing
 * (decoder/kvcache.go:21-40), or per head the int8 codes times their scale (kvcache.go:43-59 quantizeHeads / dequantHeads;
 * backend/cuda/kv8_store.cu, kvtype.cuh:48-52). */
static void kv_narrow_row(const or_model *m, const float *src, float *dst) {
    int kvDim = m->n_kv * m->head_dim;
    if (m->kv_f16 == 1) {
        for (int i = 0; i < kvDim; i++) dst[i] = or_f16_to_f32(or_f32_to_f16(src[i]));
    } else if (m->kv_f16 == 2) {
        int8_t q[1024];
        for (int h = 0; h < m->n_kv; h++) {
            float sc = or_quantize_row_int8(src + (size_t)h * m->head_dim, m->head_dim, q);
            or_dequantize_rows_int8(dst + (size_t)h * m->head_dim, q, &sc, 1, m->head_dim);
        }
    } else {
        memcpy(dst, src, sizeof(float) * (size_t)kvDim);
    }
}

void or_f16_round_trip(const float *src, float *dst, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) dst[i] = or_f16_to_f32(or_f32_to_f16(src[i]));
}

int or_cache_upload(const or_model *m, or_cache *c, int layer, int base, int n, const float *keys, const float *vals) {
    size_t kvDim = (size_t)m->n_kv * m->head_dim;
    if (layer < 0 || layer >= m->n_layers || base < 0 || n < 0 || base + n > c->cap) return -1;
    float *kd = c->k[layer] + (size_t)base * kvDim, *vd = c->v[layer] + (size_t)base * kvDim;
#pragma omp parallel for schedule(static)
    for (int i = 0; i < n; i++) {
        kv_narrow_row(m, keys + (size_t)i * kvDim, kd + (size_t)i * kvDim);
        kv_narrow_row(m, vals + (size_t)i * kvDim, vd + (size_t)i * kvDim);
    }
    if (base + n > c->pos) c->pos = base + n;
    return 0;
}

/* decoder/mlp.go:729-745 */
static void add_scaled(float *dst, const float *src, float s, int n) {
    for (int i = 0; i < n; i++) dst[i] += s * src[i];
}

/* decoder/program_cpu.go:351-364 (applyQKNorm): RMSNorm of each head with the shared [hd] weight. */
static void qk_norm(float *x, int heads, int hd, const float *w, double eps) { or_rmsnorm(x, x, w, heads, hd, eps, 0); }

/* decoder/mlp.go:36-120 (moeMLP) for one row: router matmul (M=1), routeExperts, experts in rank order,
 * out += w_j * expert_j(h) (addScaled). mlp.go:630-726 (moeMLPBatchWith) folds each row in the same rank
 * order and is bit-identical to this per-row form by its own contract. */
static void moe_mlp(const or_model *m, const or_layer *lw, const float *h, float *out, int *idx_trace, float *wts_trace, int replay) {
    int nE = m->n_experts, k = m->top_k, H = m->hidden, I = m->exp_inter;
    float *logits = (float *)malloc(sizeof(float) * (size_t)nE);
    int *idx = (int *)malloc(sizeof(int) * (size_t)k);
    float *wts = (float *)malloc(sizeof(float) * (size_t)k);
    float *g = (float *)malloc(sizeof(float) * (size_t)I), *u = (float *)malloc(sizeof(float) * (size_t)I);
    float *eo = (float *)malloc(sizeof(float) * (size_t)H);
    or_matmul(&lw->router, h, 1, logits);
    int n = or_route_experts_ex(logits, lw->router_bias, nE, k, m->router_sigmoid, m->norm_topk, m->router_scale, m->n_group, m->topk_group, idx, wts);
    if (replay) { /* decoder/mlp.go:53-56: the recorded routing replaces this call's own */
        n = k;
        for (int j = 0; j < k; j++) idx[j] = idx_trace[j], wts[j] = wts_trace[j];
    }
    memset(out, 0, sizeof(float) * (size_t)H);
    for (int j = 0; j < n; j++) {
        int e = idx[j];
        if (idx_trace && !replay) idx_trace[j] = e;
        if (wts_trace && !replay) wts_trace[j] = wts[j];
        or_matmul(&lw->exp_gate[e], h, 1, g);
        or_matmul(&lw->exp_up[e], h, 1, u);
        or_swiglu(g, u, I);
        or_matmul(&lw->exp_down[e], g, 1, eo);
        add_scaled(out, eo, wts[j], H);
    }
    free(logits);
    free(idx);
    free(wts);
    free(g);
    free(u);
    free(eo);
}

/* decoder/cpu_batch.go:166-197 (decodeMultiStep) + program_cpu_n.go:406-563 (walkMulti) + forwardn.go:800-831 (lmHeadN).
 * Pre-norm llama-style layer program: norm, q/k/v (M=B), optional QK-norm, RoPE at each row's own position,
 * per-sequence append + attention, o-proj, residual, norm, gated FFN (dense at M=B, MoE per row), residual; final norm; head. */
int or_decode_multi_step(const or_model *m, int B, const float *emb, or_cache **caches, float *logits, int *moe_idx_trace) {
    return or_decode_multi_step_traced(m, B, emb, caches, logits, moe_idx_trace, NULL, 0);
}

int or_decode_multi_step_traced(const or_model *m, int B, const float *emb, or_cache **caches, float *logits, int *moe_idx_trace,
                                float *moe_wts_trace, int replay) {
    if (replay && (!moe_idx_trace || !moe_wts_trace)) return -2;
    int H = m->hidden, nH = m->n_heads, nKV = m->n_kv, hd = m->head_dim, I = m->inter;
    int qDim = nH * hd, kvDim = nKV * hd;
    for (int b = 0; b < B; b++)
        if (caches[b]->pos >= caches[b]->cap) return -1;
    float *h = (float *)malloc(sizeof(float) * (size_t)B * H);
    float *norm = (float *)malloc(sizeof(float) * (size_t)B * H);
    float *att = (float *)malloc(sizeof(float) * (size_t)B * H);
    float *q = (float *)malloc(sizeof(float) * (size_t)B * qDim), *ctx = (float *)malloc(sizeof(float) * (size_t)B * qDim);
    float *k = (float *)malloc(sizeof(float) * (size_t)B * kvDim), *v = (float *)malloc(sizeof(float) * (size_t)B * kvDim);
    float *gate = NULL, *up = NULL;
    if (m->n_experts == 0) {
        gate = (float *)malloc(sizeof(float) * (size_t)B * I);
        up = (float *)malloc(sizeof(float) * (size_t)B * I);
    }
    memcpy(h, emb, sizeof(float) * (size_t)B * H);
    for (int l = 0; l < m->n_layers; l++) {
        const or_layer *lw = &m->layers[l];
        or_rmsnorm(norm, h, lw->attn_norm, B, H, m->eps, m->norm_add_one);
        or_matmul(&lw->q, norm, B, q);
        or_matmul(&lw->k, norm, B, k);
        or_matmul(&lw->v, norm, B, v);
        for (int b = 0; b < B; b++) {
            float *qb = q + (size_t)b * qDim, *kb = k + (size_t)b * kvDim, *vb = v + (size_t)b * kvDim;
            or_cache *c = caches[b];
            if (lw->q_bias) { /* program_cpu_n.go:470-476: addBias (attention.go:12-34) right after the projections */
                for (int i = 0; i < qDim; i++) qb[i] += lw->q_bias[i];
                for (int i = 0; i < kvDim; i++) kb[i] += lw->k_bias[i];
                for (int i = 0; i < kvDim; i++) vb[i] += lw->v_bias[i];
            }
            if (lw->q_norm) {
                qk_norm(qb, nH, hd, lw->q_norm, m->eps);
                qk_norm(kb, nKV, hd, lw->k_norm, m->eps);
            }
            const int rpos = c->pos + (g_fault == OR_FAULT_ROPE_POS ? 1 : 0); /* fault: rotated for the next position */
            or_rope(qb, nH, hd, rpos, m->inv_freq, hd / 2, 1.0);
            or_rope(kb, nKV, hd, rpos, m->inv_freq, hd / 2, 1.0);
            float *kr = c->k[l] + (size_t)c->pos * kvDim, *vr = c->v[l] + (size_t)c->pos * kvDim;
            kv_narrow_row(m, kb, kr); /* as the cache stores it: f32, binary16 or int8 per head */
            kv_narrow_row(m, vb, vr);
            /* kvmgr.WindowNeedStart (internal/runtime/kvmgr/sequence.go:55-60): a windowed layer reads keys pos-window+1 .. pos */
            const int start = lw->window > 0 && c->pos - lw->window + 1 > 0 ? c->pos - lw->window + 1 : 0;
            or_attend_sinks(qb, ctx + (size_t)b * qDim, c->k[l], c->v[l], c->pos + 1, start, nH, nKV, hd, m->attn_scale, m->softcap, lw->sinks);
        }
        or_matmul(&lw->o, ctx, B, att);
        /* Gemma 2 (decoder/program_cpu.go:286-312, the PostAttn slot): the branch output is normed before the residual add */
        if (lw->post_attn_norm) or_rmsnorm(att, att, lw->post_attn_norm, B, H, m->eps, m->norm_add_one);
        for (size_t i = 0; i < (size_t)B * H; i++) h[i] += att[i];
        or_rmsnorm(norm, h, lw->ffn_norm, B, H, m->eps, m->norm_add_one);
        if (m->n_experts == 0) {
            or_matmul(&lw->gate, norm, B, gate);
            or_matmul(&lw->up, norm, B, up);
            if (m->act_gelu_tanh) or_geglu(gate, up, B * I);
            else or_swiglu(gate, up, B * I);
            or_matmul(&lw->down, gate, B, att);
        } else {
            for (int b = 0; b < B; b++)
                moe_mlp(m, lw, norm + (size_t)b * H, att + (size_t)b * H,
                        moe_idx_trace ? moe_idx_trace + ((size_t)b * m->n_layers + l) * m->top_k : NULL,
                        moe_wts_trace ? moe_wts_trace + ((size_t)b * m->n_layers + l) * m->top_k : NULL, replay);
        }
        if (lw->post_ffn_norm) or_rmsnorm(att, att, lw->post_ffn_norm, B, H, m->eps, m->norm_add_one);
        for (size_t i = 0; i < (size_t)B * H; i++) h[i] += att[i];
    }
    for (int b = 0; b < B; b++) caches[b]->pos++;
    or_rmsnorm(h, h, m->final_norm, B, H, m->eps, m->norm_add_one);
    or_matmul(&m->head, h, B, logits);
    if (m->final_softcap > 0) or_softcap_logits(logits, (size_t)B * m->vocab, (float)m->final_softcap);
    if (m->logit_scale != 0 && m->logit_scale != 1) { /* decoder/model_forward.go:304-320, forwardn.go:823-831 */
        const float inv = (float)(1 / m->logit_scale);
        for (size_t i = 0; i < (size_t)B * m->vocab; i++) logits[i] *= inv;
    }
    free(h);
    free(norm);
    free(att);
    free(q);
    free(ctx);
    free(k);
    free(v);
    free(gate);
    free(up);
    return 0;
}
