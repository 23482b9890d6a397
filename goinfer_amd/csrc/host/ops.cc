// ops.cc — the kernel-level entry points (host pointers in, host pointers out): what the reference's kernel tests bind
// (backend/cuda/kernels/actgroup_kernel_test.go, flash_decode_test.go, moe_route_test.go) and what the micro-benchmarks time.
#include "device.h"
#include <algorithm>
#include <vector>
#include <cmath>
#include <numeric>
#include <string.h>
#include <string>

#define RC(x)                \
    do {                     \
        int rd_rc_macro_ = (x); \
        if (rd_rc_macro_) return rd_rc_macro_; \
    } while (0)

extern "C" int rd_dequant_q4k(rd_device *d, const void *blocks, int N, int K, float *out) {
    if (!d || !blocks || !out || N <= 0 || K <= 0 || K % 256) {
        rd_set_error("rd_dequant_q4k: bad arguments (K must be a multiple of 256)");
        return RD_ERR_ARG;
    }
    size_t nb = (size_t)N * (K / 256);
    DevBuf raw(d), o(d);
    RC(raw.alloc(nb * 144));
    RC(o.alloc(nb * 256 * sizeof(float)));
    RC(d->h2d(raw.p, blocks, nb * 144));
    RC(d->launch(d->k.dequant_q4k, (unsigned)nb, 1, 1, 256, (const void *)raw.p, o.as<float>(), (long)nb));
    return d->d2h(out, o.p, nb * 256 * sizeof(float));
}

// a[M][K] on the device (M <= 32) -> quantized panels of `kind`, per 32 or (act_group 0) per row.
static int quantize_rows(rd_device *d, const float *a_dev, int M, int K, int kind, int act_group, void *Xp) {
    return launch_quant_act(d, a_dev, M, K, kind, act_group, Xp);
}

static int gemm_host(rd_device *d, DevWeight &w, DevWeight *w2, const float *a, int M, float *dst) {
    int N = w.N, K = w.K;
    size_t pbytes = panel_bytes_for(w);
    int kind = panel_kind_for(w);
    const int chunk = w2 ? 32 : GEMM_WIDE_ROWS, tiles = chunk / 32; // rows per pass: M-tiles of 32 side by side
    DevBuf A(d), Xp(d), P(d), O(d);
    RC(A.alloc(sizeof(float) * (size_t)chunk * K));
    RC(Xp.alloc(pbytes * tiles));
    int nKB = kblocks_for(w);
    int Ntot = w2 ? 2 * N : N;
    int maxSplits = plan_gemm(w.kind, Ntot, nKB, w.act_group).splits;
    const size_t pStride = (size_t)maxSplits * 32 * Ntot;
    RC(P.alloc(sizeof(float) * pStride * tiles));
    RC(O.alloc(sizeof(float) * (size_t)chunk * N));
    for (int m0 = 0; m0 < M; m0 += chunk) {
        int mc = std::min(chunk, M - m0);
        RC(d->h2d(A.p, a + (size_t)m0 * K, sizeof(float) * (size_t)mc * K));
        for (int t = 0; t * 32 < mc; t++)
            RC(quantize_rows(d, A.as<float>() + (size_t)t * 32 * K, std::min(32, mc - t * 32), K, kind, w.act_group, (char *)Xp.p + (size_t)t * pbytes));
        GemmPlan plan;
        if (!w2) {
            RC(launch_gemm_wide(d, w, Xp.p, pbytes, P.as<float>(), pStride, mc, &plan));
            for (int t = 0; t * 32 < mc; t++)
                RC(d->launch(d->k.reduce_splits, (unsigned)((N + 255) / 256), (unsigned)std::min(32, mc - t * 32), 1, 256,
                             (const float *)(P.as<float>() + (size_t)t * pStride), O.as<float>() + (size_t)t * 32 * N, N, plan.splits));
        } else {
            // gate|up stacked (2N rows): GEMM, then SwiGLU over the reduced partial sums
            RC(launch_gemm(d, *w2, Xp.p, P.as<float>(), mc, &plan));
            DevBuf X2(d);
            RC(X2.alloc(a8_bytes(N)));
            RC(d->launch(d->k.swiglu_quant, (unsigned)((N + 1023) / 1024), (unsigned)mc, 1, 256, (const float *)P.p, plan.splits, N, X2.p,
                         (int)PANEL_A8, O.as<float>(), (size_t)0, (size_t)0, 0));
            RC(d->sync());
        }
        RC(d->d2h(dst + (size_t)m0 * N, O.p, sizeof(float) * (size_t)mc * N));
    }
    return RD_OK;
}

extern "C" int rd_gemm_q4k(rd_device *d, const void *W, int N, int K, const float *a, int M, float *dst, const void *W2) {
    if (!d || !W || !a || !dst || M <= 0) {
        rd_set_error("rd_gemm_q4k: bad arguments");
        return RD_ERR_ARG;
    }
    DevWeight w, wcat;
    int rc;
    if (!W2) {
        if ((rc = upload_q4k(d, W, N, K, &w))) return rc;
        rc = gemm_host(d, w, nullptr, a, M, dst);
        free_weight(d, &w);
        return rc;
    }
    if (N % 256) { // the SwiGLU output feeds a Q4_K-style panel writer in chunks of 256
        rd_set_error("rd_gemm_q4k fused: N=%d must be a multiple of 256", N);
        return RD_DECLINED;
    }
    size_t bytes = (size_t)N * (K / 256) * 144;
    std::vector<uint8_t> cat(2 * bytes);
    memcpy(cat.data(), W, bytes);
    memcpy(cat.data() + bytes, W2, bytes);
    if ((rc = upload_q4k(d, cat.data(), 2 * N, K, &wcat))) return rc;
    w.kind = 0, w.N = N, w.K = K;
    rc = gemm_host(d, w, &wcat, a, M, dst);
    free_weight(d, &wcat);
    return rc;
}

extern "C" int rd_gateup_q4k_quant(rd_device *d, const void *Wg, const void *Wu, int I, int K, const float *a, int M, float *dst) {
    if (!d || !Wg || !Wu || !a || !dst || M <= 0) {
        rd_set_error("rd_gateup_q4k_quant: bad arguments");
        return RD_ERR_ARG;
    }
    if (I <= 0 || I % 256 || K <= 0 || K % 256) {
        rd_set_error("rd_gateup_q4k_quant: I=%d and K=%d must be multiples of 256", I, K);
        return RD_DECLINED;
    }
    size_t bytes = (size_t)I * (K / 256) * 144;
    std::vector<uint8_t> cat(2 * bytes);
    memcpy(cat.data(), Wg, bytes);
    memcpy(cat.data() + bytes, Wu, bytes);
    DevWeight w;
    int rc = upload_q4k(d, cat.data(), 2 * I, K, &w);
    if (rc) return rc;
    DevBuf A(d), Xp(d), X2(d), O(d);
    auto body = [&]() -> int {
        // passes of up to GEMM_WIDE_ROWS rows as the step runs them: up to 32 rows in the decode kernel, more in the many-row kernel
        const int chunk = std::min(M, GEMM_WIDE_ROWS), tiles = (chunk + 31) / 32;
        const size_t xpStride = a8_bytes(K), x2Stride = a8_bytes(I);
        RC(A.alloc(sizeof(float) * (size_t)chunk * K));
        RC(Xp.alloc(xpStride * tiles));
        RC(X2.alloc(x2Stride * tiles));
        RC(O.alloc(sizeof(float) * (size_t)chunk * I));
        for (int m0 = 0; m0 < M; m0 += chunk) {
            int mc = std::min(chunk, M - m0);
            RC(d->h2d(A.p, a + (size_t)m0 * K, sizeof(float) * (size_t)mc * K));
            for (int t = 0; t * 32 < mc; t++)
                RC(quantize_rows(d, A.as<float>() + (size_t)t * 32 * K, std::min(32, mc - t * 32), K, PANEL_A8, 32, (char *)Xp.p + (size_t)t * xpStride));
            if (mc >= ROWS_GEMM_MIN_ROWS && rows_gemm_enabled())
                RC(d->launch(d->k.gemm8_q4k_rows_gateup, (unsigned)(I / 32), 1, (unsigned)((mc + 127) / 128), 256, (const void *)w.tiled, (const void *)Xp.p,
                             X2.as<uint8_t>(), I, K / 256, mc, xpStride, x2Stride));
            else
                RC(d->launch(d->k.gemm8_q4k_gateup, (unsigned)(I / 32), 1, (unsigned)((mc + 31) / 32), GATEUP_THREADS, (const void *)w.tiled, (const void *)Xp.p,
                             X2.as<uint8_t>(), (int)PANEL_A8, I, K / 256, mc, xpStride, x2Stride));
            for (int t = 0; t * 32 < mc; t++)
                RC(d->launch(d->k.unpanel_a8, (unsigned)(I / 256), (unsigned)std::min(32, mc - t * 32), 1, 256, (const void *)((char *)X2.p + (size_t)t * x2Stride),
                             O.as<float>() + (size_t)t * 32 * I, I));
            RC(d->d2h(dst + (size_t)m0 * I, O.p, sizeof(float) * (size_t)mc * I));
        }
        return RD_OK;
    };
    rc = body();
    free_weight(d, &w);
    return rc;
}

// The activation quantizer on its own (goinfer: aikit QuantizeActQ, call sites decoder/weightmat.go:845-862;
// backend/cuda/actgroup.cu:32-54 quantG32, kv8_store.cu:27-35 for the per-row rule): a f32 [M][K] -> int8 codes [M][K] and,
// act_group 32: f32 scales and sums (scale * sum of codes) [M][K/32]; act_group 0: one scale per row, scales [M] (sums untouched,
// may be NULL). As the GEMMs consume them. K % 32 == 0.
extern "C" int rd_quant_act(rd_device *d, const float *a, int M, int K, int act_group, int8_t *codes, float *scales, float *sums) {
    if (!d || !a || !codes || !scales || (!sums && act_group != 0) || M <= 0 || K <= 0 || K % 32 || (act_group != 0 && act_group != 32)) {
        rd_set_error("rd_quant_act: bad arguments (K must be a multiple of 32, act_group 32 or 0)");
        return RD_ERR_ARG;
    }
    const int nG = K / 32;
    std::vector<float> rowS((size_t)32 * nG);
    DevBuf A(d), A8(d), C(d), S(d), U(d);
    RC(A.alloc(sizeof(float) * (size_t)32 * K));
    RC(A8.alloc(a8_bytes(K)));
    RC(C.alloc((size_t)32 * K));
    RC(S.alloc(sizeof(float) * (size_t)32 * nG));
    RC(U.alloc(sizeof(float) * (size_t)32 * nG));
    for (int m0 = 0; m0 < M; m0 += 32) {
        const int mc = std::min(32, M - m0);
        RC(d->h2d(A.p, a + (size_t)m0 * K, sizeof(float) * (size_t)mc * K));
        RC(quantize_rows(d, A.as<float>(), mc, K, PANEL_A8, act_group, A8.p));
        RC(d->launch(d->k.unpack_act8, (unsigned)((K + 255) / 256), (unsigned)mc, 1, 256, (const void *)A8.p, (signed char *)C.p, S.as<float>(), U.as<float>(), K));
        RC(d->d2h(codes + (size_t)m0 * K, C.p, (size_t)mc * K));
        if (act_group == 0) { // the row's scale sits in every group slot: the first is returned
            RC(d->d2h(rowS.data(), S.p, sizeof(float) * (size_t)mc * nG));
            for (int r = 0; r < mc; r++) scales[m0 + r] = rowS[(size_t)r * nG];
            continue;
        }
        RC(d->d2h(scales + (size_t)m0 * nG, S.p, sizeof(float) * (size_t)mc * nG));
        RC(d->d2h(sums + (size_t)m0 * nG, U.p, sizeof(float) * (size_t)mc * nG));
    }
    return RD_OK;
}

// Q5_K / Q6_K: the file's own super-blocks (176 B / 210 B per 256 weights) dequantized or multiplied natively.
static int dequant_kquant(rd_device *d, hipFunction_t k, int bb, const void *blocks, int N, int K, float *out, const char *who) {
    if (!d || !blocks || !out || N <= 0 || K <= 0 || K % 256) {
        rd_set_error("%s: bad arguments (K must be a multiple of 256)", who);
        return RD_ERR_ARG;
    }
    size_t nb = (size_t)N * (K / 256);
    DevBuf raw(d), o(d);
    RC(raw.alloc(nb * bb));
    RC(o.alloc(nb * 256 * sizeof(float)));
    RC(d->h2d(raw.p, blocks, nb * bb));
    RC(d->launch(k, (unsigned)nb, 1, 1, 256, (const void *)raw.p, o.as<float>(), (long)nb));
    return d->d2h(out, o.p, nb * 256 * sizeof(float));
}
extern "C" int rd_dequant_q5k(rd_device *d, const void *blocks, int N, int K, float *out) {
    return dequant_kquant(d, d ? d->k.dequant_q5k : nullptr, 176, blocks, N, K, out, "rd_dequant_q5k");
}
extern "C" int rd_dequant_q6k(rd_device *d, const void *blocks, int N, int K, float *out) {
    return dequant_kquant(d, d ? d->k.dequant_q6k : nullptr, 210, blocks, N, K, out, "rd_dequant_q6k");
}
extern "C" int rd_gemm_q5k(rd_device *d, const void *W, int N, int K, const float *a, int M, float *dst) {
    if (!d || !W || !a || !dst || M <= 0) {
        rd_set_error("rd_gemm_q5k: bad arguments");
        return RD_ERR_ARG;
    }
    DevWeight w;
    int rc = upload_q5k(d, W, N, K, &w);
    if (rc) return rc;
    rc = gemm_host(d, w, nullptr, a, M, dst);
    free_weight(d, &w);
    return rc;
}
extern "C" int rd_gemm_q6k(rd_device *d, const void *W, int N, int K, const float *a, int M, float *dst) {
    if (!d || !W || !a || !dst || M <= 0) {
        rd_set_error("rd_gemm_q6k: bad arguments");
        return RD_ERR_ARG;
    }
    DevWeight w;
    int rc = upload_q6k(d, W, N, K, &w);
    if (rc) return rc;
    rc = gemm_host(d, w, nullptr, a, M, dst);
    free_weight(d, &w);
    return rc;
}

extern "C" int rd_gemm_w8a8(rd_device *d, const int8_t *q, const float *row_scale, int N, int K, const float *a, int M, int act_group, float *dst) {
    if (!d || !q || !row_scale || !a || !dst || M <= 0) return RD_ERR_ARG;
    DevWeight w;
    int rc = upload_w8a8(d, q, row_scale, N, K, &w, act_group);
    if (rc) return rc;
    rc = gemm_host(d, w, nullptr, a, M, dst);
    free_weight(d, &w);
    return rc;
}

extern "C" int rd_gemm_w4a8(rd_device *d, const uint8_t *nib, const uint16_t *s16, int N, int K, const float *a, int M, int act_group, float *dst) {
    if (!d || !nib || !s16 || !a || !dst || M <= 0) return RD_ERR_ARG;
    DevWeight w;
    int rc = upload_w4a8(d, nib, s16, N, K, &w, false, act_group);
    if (rc) return rc;
    rc = gemm_host(d, w, nullptr, a, M, dst);
    free_weight(d, &w);
    return rc;
}

// Device-side draws over explicit logit rows: the kernels the step ends with, on their own (what the reference's
// backend/cuda/kernels/gumbel_test.go binds). Rows are padded to a multiple of four columns with -Inf, which is never drawn.
extern "C" int rd_sample_rows(rd_device *d, const float *logits, int rows, int V, const rd_draw *draws, int *ids) {
    if (!d || !logits || !draws || !ids || rows <= 0 || V <= 0) {
        rd_set_error("rd_sample_rows: bad arguments");
        return RD_ERR_ARG;
    }
    const int Vp = (V + 3) & ~3, nChunks = (Vp + 4095) / 4096;
    DevBuf L(d), cv(d), ci(d), rec(d), out(d);
    RC(L.alloc(sizeof(float) * (size_t)32 * Vp));
    RC(cv.alloc(sizeof(float) * (size_t)32 * nChunks));
    RC(ci.alloc(sizeof(int) * (size_t)32 * nChunks));
    RC(rec.alloc(sizeof(int) * 32 * 6));
    RC(out.alloc(sizeof(int) * 32));
    std::vector<float> pad((size_t)32 * Vp);
    for (int r0 = 0; r0 < rows; r0 += 32) {
        int nr = std::min(32, rows - r0);
        int recs[32 * 6] = {0};
        for (int r = 0; r < nr; r++) {
            const rd_draw &dw = draws[r0 + r];
            int *q = recs + r * 6;
            q[0] = dw.mode == RD_DRAW_NONE ? RD_DRAW_GREEDY : dw.mode;
            if (dw.mode == RD_DRAW_GUMBEL) {
                float invT = (float)(1.0 / (dw.temperature <= 0 ? 1.0 : dw.temperature));
                if (std::isinf(invT)) {
                    q[0] = RD_DRAW_GREEDY;
                } else {
                    memcpy(&q[1], &invT, 4);
                    q[2] = (int)(uint32_t)dw.seed, q[3] = (int)(uint32_t)(dw.seed >> 32), q[4] = (int)(uint32_t)dw.draw, q[5] = (int)(uint32_t)(dw.draw >> 32);
                }
            }
            memcpy(pad.data() + (size_t)r * Vp, logits + (size_t)(r0 + r) * V, sizeof(float) * (size_t)V);
            for (int c = V; c < Vp; c++) pad[(size_t)r * Vp + c] = -INFINITY;
        }
        RC(d->h2d(L.p, pad.data(), sizeof(float) * (size_t)nr * Vp));
        RC(d->h2d(rec.p, recs, sizeof(recs)));
        RC(d->launch(d->k.argmax_rows, (unsigned)nChunks, (unsigned)nr, 1, 256, (const float *)L.p, 1, Vp, cv.as<float>(), ci.as<int>(), (float *)nullptr,
                     (const int *)rec.p, (size_t)0, 0.f, 0.f));
        RC(d->launch(d->k.argmax_final, (unsigned)nr, 1, 1, 64, (const float *)cv.p, (const int *)ci.p, nChunks, out.as<int>()));
        RC(d->d2h(ids + r0, out.p, sizeof(int) * (size_t)nr));
    }
    return RD_OK;
}

extern "C" int rd_matmul_bt(rd_device *d, const float *a, const float *b, float *dst, int M, int K, int N) {
    if (!d || !a || !b || !dst || M <= 0 || K <= 0 || N <= 0) return RD_ERR_ARG;
    DevBuf A(d), B(d), D(d);
    RC(A.alloc(sizeof(float) * (size_t)M * K));
    RC(B.alloc(sizeof(float) * (size_t)N * K));
    RC(D.alloc(sizeof(float) * (size_t)M * N));
    RC(d->h2d(A.p, a, sizeof(float) * (size_t)M * K));
    RC(d->h2d(B.p, b, sizeof(float) * (size_t)N * K));
    RC(d->launch(d->k.matmul_f32, (unsigned)((N + 3) / 4), (unsigned)M, 1, 256, (const float *)A.p, (const float *)B.p, D.as<float>(), M, K, N, (unsigned *)nullptr, (unsigned *)nullptr, 0));
    return d->d2h(dst, D.p, sizeof(float) * (size_t)M * N);
}

extern "C" int rd_rmsnorm(rd_device *d, const float *x, const float *w, int rows, int dim, float eps, float *out) {
    if (!d || !x || !w || !out || rows <= 0 || dim <= 0) return RD_ERR_ARG;
    DevBuf X(d), W(d), O(d);
    RC(X.alloc(sizeof(float) * (size_t)rows * dim));
    RC(W.alloc(sizeof(float) * (size_t)dim));
    RC(O.alloc(sizeof(float) * (size_t)rows * dim));
    RC(d->h2d(X.p, x, sizeof(float) * (size_t)rows * dim));
    RC(d->h2d(W.p, w, sizeof(float) * (size_t)dim));
    RC(d->launch(d->k.rmsnorm, (unsigned)rows, 1, 1, 256, (const float *)X.p, (const float *)W.p, O.as<float>(), dim, eps));
    return d->d2h(out, O.p, sizeof(float) * (size_t)rows * dim);
}

extern "C" int rd_rope(rd_device *d, float *vec, int rows, int heads, int head_dim, const int *pos, const double *inv_freq) {
    if (!d || !vec || !pos || !inv_freq || rows <= 0 || heads <= 0 || head_dim <= 0 || head_dim % 2 || head_dim > 2048) return RD_ERR_ARG;
    size_t n = (size_t)rows * heads * head_dim;
    DevBuf V(d), Pp(d), F(d);
    RC(V.alloc(sizeof(float) * n));
    RC(Pp.alloc(sizeof(int) * (size_t)rows));
    RC(F.alloc(sizeof(double) * (size_t)(head_dim / 2)));
    RC(d->h2d(V.p, vec, sizeof(float) * n));
    RC(d->h2d(Pp.p, pos, sizeof(int) * (size_t)rows));
    RC(d->h2d(F.p, inv_freq, sizeof(double) * (size_t)(head_dim / 2)));
    RC(d->launch(d->k.rope, (unsigned)heads, (unsigned)rows, 1, (unsigned)(head_dim / 2), V.as<float>(), (const int *)Pp.p, (const double *)F.p, heads,
                 head_dim));
    return d->d2h(vec, V.p, sizeof(float) * n);
}

extern "C" int rd_moe_route_ex(rd_device *d, const float *logits, const float *bias, int T, int nE, int k, int sigmoid, int norm, double scale,
                               int n_group, int topk_group, int *idx, float *wgt) {
    if (!d || !logits || !idx || !wgt || T <= 0 || nE <= 0 || nE > 256 || k <= 0 || k > nE) {
        rd_set_error("rd_moe_route: bad arguments (nE <= 256)");
        return RD_ERR_ARG;
    }
    if (n_group > 32 || (n_group > 1 && (topk_group < 1 || topk_group > n_group))) {
        rd_set_error("rd_moe_route: group-limited routing takes 2..32 groups and 1..n_group of them");
        return RD_ERR_ARG;
    }
    DevBuf L(d), I(d), W(d), Bi(d);
    RC(L.alloc(sizeof(float) * (size_t)T * nE));
    RC(I.alloc(sizeof(int) * (size_t)T * k));
    RC(W.alloc(sizeof(float) * (size_t)T * k));
    RC(d->h2d(L.p, logits, sizeof(float) * (size_t)T * nE));
    RC(d->launch(d->k.fill_f32, 1, 1, 1, 64, I.as<float>(), (size_t)T * k, 0u)); // a row with fewer than k eligible experts leaves the rest as it finds it
    if (bias) {
        RC(Bi.alloc(sizeof(float) * (size_t)nE));
        RC(d->h2d(Bi.p, bias, sizeof(float) * (size_t)nE));
    }
    RC(d->launch(d->k.moe_route, (unsigned)T, 1, 1, 64, (const float *)L.p, T, nE, k, norm, I.as<int>(), W.as<float>(),
                 (signed char *)nullptr, (int *)nullptr, (unsigned *)nullptr, (const float *)Bi.p, sigmoid, (float)scale, n_group, topk_group));
    RC(d->d2h(idx, I.p, sizeof(int) * (size_t)T * k));
    return d->d2h(wgt, W.p, sizeof(float) * (size_t)T * k);
}
extern "C" int rd_moe_route(rd_device *d, const float *logits, int T, int nE, int k, int norm, int *idx, float *wgt) {
    return rd_moe_route_ex(d, logits, nullptr, T, nE, k, 0, norm, 0.0, 0, 0, idx, wgt);
}

// ---- the step's q|k|v epilogue on its own: bias, QK-norm, RoPE, and the K/V rows as the cache then holds them ----
// x: f32 [rows][(n_h + 2 n_kv) * hd], the q|k|v projection outputs of `rows` sequences, row r at position pos[r] of its own
// one-sequence cache. q_out: f32 [rows][n_h*hd]; k_out, v_out: f32 [rows][n_kv*hd], read back from the cache (f16 widened, or
// code * scale for the int8 cache). q_norm, k_norm, bias may be null.
extern "C" int rd_qkv_rope_store(rd_device *d, int kv_type, int rows, const float *x, const int *pos, int n_h, int n_kv, int hd, const double *inv_freq,
                                 const float *q_norm, const float *k_norm, float eps, const float *bias, float *q_out, float *k_out, float *v_out) {
    if (!d || !x || !pos || !inv_freq || !q_out || !k_out || !v_out || rows <= 0 || rows > 32) {
        rd_set_error("rd_qkv_rope_store: bad arguments (1 <= rows <= 32)");
        return RD_ERR_ARG;
    }
    if (n_h <= 0 || n_kv <= 0 || (hd != 64 && hd != 128) || (kv_type != RD_KV_F16 && kv_type != RD_KV_I8)) {
        rd_set_error("rd_qkv_rope_store declines: head_dim must be 64 or 128");
        return RD_DECLINED;
    }
    int maxPos = 0;
    for (int r = 0; r < rows; r++) {
        if (pos[r] < 0) return RD_ERR_ARG;
        maxPos = std::max(maxPos, pos[r]);
    }
    const bool i8 = kv_type == RD_KV_I8;
    const int bps = maxPos / 64 + 1, Ntot = (n_h + 2 * n_kv) * hd, kvd = n_kv * hd;
    const size_t nBlocks = (size_t)rows * bps + 1;
    const size_t poolBytes = nBlocks * n_kv * 64 * hd * (i8 ? 1 : 2), scBytes = nBlocks * n_kv * 64 * sizeof(float);
    std::vector<int> tab((size_t)rows * bps), slots((size_t)rows);
    for (size_t i = 0; i < tab.size(); i++) tab[i] = (int)i + 1;
    for (int r = 0; r < rows; r++) slots[(size_t)r] = r;
    DevBuf X(d), Q(d), Kp(d), Vp(d), Ksc(d), Vsc(d), T(d), S(d), Pp(d), F(d), QN(d), KN(d), Bi(d), Ko(d), Vo(d);
    RC(X.alloc(sizeof(float) * (size_t)32 * Ntot));
    RC(Q.alloc(sizeof(float) * (size_t)rows * n_h * hd));
    RC(Kp.alloc(poolBytes));
    RC(Vp.alloc(poolBytes));
    HIPCHK(MemsetAsync(Kp.p, 0, poolBytes, d->stream));
    HIPCHK(MemsetAsync(Vp.p, 0, poolBytes, d->stream));
    RC(Ksc.alloc(scBytes));
    RC(Vsc.alloc(scBytes));
    HIPCHK(MemsetAsync(Ksc.p, 0, scBytes, d->stream));
    HIPCHK(MemsetAsync(Vsc.p, 0, scBytes, d->stream));
    RC(T.alloc(sizeof(int) * tab.size()));
    RC(S.alloc(sizeof(int) * (size_t)rows));
    RC(Pp.alloc(sizeof(int) * (size_t)rows));
    RC(F.alloc(sizeof(double) * (size_t)(hd / 2)));
    RC(Ko.alloc(sizeof(float) * (size_t)kvd));
    RC(Vo.alloc(sizeof(float) * (size_t)kvd));
    RC(d->h2d(X.p, x, sizeof(float) * (size_t)rows * Ntot));
    RC(d->h2d(T.p, tab.data(), sizeof(int) * tab.size()));
    RC(d->h2d(S.p, slots.data(), sizeof(int) * (size_t)rows));
    RC(d->h2d(Pp.p, pos, sizeof(int) * (size_t)rows));
    RC(d->h2d(F.p, inv_freq, sizeof(double) * (size_t)(hd / 2)));
    if (q_norm) {
        RC(QN.alloc(sizeof(float) * (size_t)hd));
        RC(d->h2d(QN.p, q_norm, sizeof(float) * (size_t)hd));
    }
    if (k_norm) {
        RC(KN.alloc(sizeof(float) * (size_t)hd));
        RC(d->h2d(KN.p, k_norm, sizeof(float) * (size_t)hd));
    }
    if (bias) {
        RC(Bi.alloc(sizeof(float) * (size_t)Ntot));
        RC(d->h2d(Bi.p, bias, sizeof(float) * (size_t)Ntot));
    }
    if (i8)
        RC(d->launch(d->k.qkv_rope_store_i8, (unsigned)(n_h + 2 * n_kv), (unsigned)rows, 1, (unsigned)(hd / 2), (const float *)X.p, 1, Q.as<float>(),
                     (signed char *)Kp.p, (signed char *)Vp.p, Ksc.as<float>(), Vsc.as<float>(), (const int *)T.p, bps, (const int *)S.p, (const int *)Pp.p,
                     (const double *)F.p, (const float *)QN.p, (const float *)KN.p, eps, n_h, n_kv, hd, (size_t)0, (const float *)Bi.p, 0));
    else
        RC(d->launch(d->k.qkv_rope_store, (unsigned)(n_h + 2 * n_kv), (unsigned)rows, 1, (unsigned)(hd / 2), (const float *)X.p, 1, Q.as<float>(),
                     (uint16_t *)Kp.p, (uint16_t *)Vp.p, (const int *)T.p, bps, (const int *)S.p, (const int *)Pp.p, (const double *)F.p, (const float *)QN.p,
                     (const float *)KN.p, eps, n_h, n_kv, hd, (size_t)0, (const float *)Bi.p, 0));
    RC(d->d2h(q_out, Q.p, sizeof(float) * (size_t)rows * n_h * hd));
    for (int r = 0; r < rows; r++) {
        RC(d->launch(d->k.kv_read, 1u, (unsigned)n_kv, 1, (unsigned)hd, (const void *)Kp.p, (const void *)Vp.p, (const float *)Ksc.p, (const float *)Vsc.p,
                     Ko.as<float>(), Vo.as<float>(), (const int *)((const int *)T.p + (size_t)r * bps), pos[r], n_kv, hd, i8 ? 1 : 0));
        RC(d->d2h(k_out + (size_t)r * kvd, Ko.p, sizeof(float) * (size_t)kvd));
        RC(d->d2h(v_out + (size_t)r * kvd, Vo.p, sizeof(float) * (size_t)kvd));
    }
    return RD_OK;
}

// ---- ragged attention over a temporary paged pool (kernel-level entry point) ----
// nq (optional): sequence i brings nq[i] query rows, its last nq[i] positions; row j of them sees keys 0..len[i]-nq[i]+j.
static int attn_ragged_typed(rd_device *d, int kv_type, int n_seq, const int *len, const int *nq, const int64_t *off, const float *k, const float *v,
                             const float *q, int n_h, int n_kv, int hd, float scale, float softcap, float *out, int window = 0, const float *sinks = nullptr) {
    if (!d || !len || !off || !k || !v || !q || !out || n_seq <= 0) return RD_ERR_ARG;
    if (n_kv <= 0 || n_h % n_kv || n_h / n_kv > 16 || (hd != 64 && hd != 128)) {
        rd_set_error("rd_attn_ragged declines: head_dim must be 64 or 128 and the GQA group <= 16");
        return RD_DECLINED;
    }
    int kvd = n_kv * hd, qd = n_h * hd, G = n_h / n_kv;
    int maxBlocks = 0;
    long totalBlocks = 0;
    for (int i = 0; i < n_seq; i++) {
        if (len[i] <= 0) {
            rd_set_error("sequence %d has no keys", i);
            return RD_ERR_ARG;
        }
        if (nq && (nq[i] <= 0 || nq[i] > len[i])) {
            rd_set_error("sequence %d: %d query rows over %d keys", i, nq[i], len[i]);
            return RD_ERR_ARG;
        }
        int nb = (len[i] + 63) / 64;
        maxBlocks = std::max(maxBlocks, nb), totalBlocks += nb;
    }
    // Scattered block table: physical blocks are handed out in a stride permutation, so paging is exercised.
    std::vector<int> tab((size_t)n_seq * maxBlocks, 0);
    {
        long nb = totalBlocks, stride = std::max(1L, (long)(nb * 0.618));
        while (stride < nb && std::gcd(stride, nb) != 1) stride++;
        if (stride >= nb) stride = 1;
        long idx = 0;
        for (int i = 0; i < n_seq; i++)
            for (int b = 0; b < (len[i] + 63) / 64; b++, idx++) tab[(size_t)i * maxBlocks + b] = 1 + (int)((idx * stride) % nb);
    }
    const bool i8 = kv_type == RD_KV_I8;
    size_t poolBytes = (size_t)(totalBlocks + 1) * n_kv * 64 * hd * (i8 ? 1 : 2), scBytes = (size_t)(totalBlocks + 1) * n_kv * 64 * sizeof(float);
    DevBuf Kp(d), Vp(d), Ksc(d), Vsc(d), T(d), Q(d), O(d), L(d), S(d), It(d), St(d), Part(d);
    RC(Kp.alloc(poolBytes));
    RC(Vp.alloc(poolBytes));
    HIPCHK(MemsetAsync(Kp.p, 0, poolBytes, d->stream));
    HIPCHK(MemsetAsync(Vp.p, 0, poolBytes, d->stream));
    if (i8) {
        RC(Ksc.alloc(scBytes));
        RC(Vsc.alloc(scBytes));
        HIPCHK(MemsetAsync(Ksc.p, 0, scBytes, d->stream));
        HIPCHK(MemsetAsync(Vsc.p, 0, scBytes, d->stream));
    }
    RC(T.alloc(sizeof(int) * tab.size()));
    RC(d->h2d(T.p, tab.data(), sizeof(int) * tab.size()));
    {
        int chunkRows = 4096;
        DevBuf Kc(d), Vc(d);
        RC(Kc.alloc(sizeof(float) * (size_t)chunkRows * kvd));
        RC(Vc.alloc(sizeof(float) * (size_t)chunkRows * kvd));
        for (int i = 0; i < n_seq; i++)
            for (int base = 0; base < len[i]; base += chunkRows) {
                int n = std::min(chunkRows, len[i] - base);
                RC(d->h2d(Kc.p, k + ((size_t)off[i] + base) * kvd, sizeof(float) * (size_t)n * kvd));
                RC(d->h2d(Vc.p, v + ((size_t)off[i] + base) * kvd, sizeof(float) * (size_t)n * kvd));
                if (i8)
                    RC(d->launch(d->k.kv_store_i8, (unsigned)n, (unsigned)n_kv, 1, 64, (const float *)Kc.p, (const float *)Vc.p, (signed char *)Kp.p,
                                 (signed char *)Vp.p, Ksc.as<float>(), Vsc.as<float>(), (const int *)((const int *)T.p + (size_t)i * maxBlocks), base, n_kv, hd));
                else
                    RC(d->launch(d->k.kv_store, (unsigned)n, (unsigned)n_kv, 1, (unsigned)hd, (const float *)Kc.p, (const float *)Vc.p, (uint16_t *)Kp.p,
                                 (uint16_t *)Vp.p, (const int *)((const int *)T.p + (size_t)i * maxBlocks), base, n_kv, hd));
                RC(d->sync());
            }
    }
    std::vector<int> rowSeq, rowLens; // the query rows in order: sequence, keys visible
    for (int i = 0; i < n_seq; i++)
        for (int j = 0, n = nq ? nq[i] : 1; j < n; j++) rowSeq.push_back(i), rowLens.push_back(len[i] - n + 1 + j);
    const int n_rows = (int)rowSeq.size();
    for (int r0 = 0; r0 < n_rows; r0 += 32) { // rows in groups of 32, as the step batches them
        int rows = std::min(32, n_rows - r0);
        std::vector<AttnItemH> items;
        std::vector<int> start, slots(rowSeq.begin() + r0, rowSeq.begin() + r0 + rows), lens(rowLens.begin() + r0, rowLens.begin() + r0 + rows);
        const bool grouped = build_attn_worklist(lens.data(), nq ? slots.data() : nullptr, G, rows, n_kv, items, start, window);
        attn_pad_items(items); // launched as the step launches it
        const int partRows = grouped ? ATTN_TILE_ROWS : G;
        DevBuf Q2(d), O2(d), L2(d), S2(d), I2(d), St2(d), P2(d), Sk(d);
        if (sinks) {
            RC(Sk.alloc(sizeof(float) * (size_t)n_h));
            RC(d->h2d(Sk.p, sinks, sizeof(float) * (size_t)n_h));
        }
        RC(Q2.alloc(sizeof(float) * (size_t)rows * qd));
        RC(O2.alloc(sizeof(float) * (size_t)rows * qd));
        RC(L2.alloc(sizeof(int) * (size_t)rows));
        RC(S2.alloc(sizeof(int) * (size_t)rows));
        RC(I2.alloc(sizeof(AttnItemH) * items.size()));
        RC(St2.alloc(sizeof(int) * start.size()));
        RC(P2.alloc(sizeof(float) * items.size() * partRows * (hd + 2)));
        RC(d->h2d(Q2.p, q + (size_t)r0 * qd, sizeof(float) * (size_t)rows * qd));
        RC(d->h2d(L2.p, lens.data(), sizeof(int) * (size_t)rows));
        RC(d->h2d(S2.p, slots.data(), sizeof(int) * (size_t)rows));
        RC(d->h2d(I2.p, items.data(), sizeof(AttnItemH) * items.size()));
        RC(d->h2d(St2.p, start.data(), sizeof(int) * start.size()));
        const AttnLaunch al = attn_partial_kernel(d, i8, grouped, items.size());
        if (i8)
            RC(d->launch(al.f, (unsigned)(items.size() / al.waves), 1, 1, 64 * al.waves, (const void *)I2.p, (const int *)L2.p,
                         (const int *)S2.p, (const int *)T.p, maxBlocks, (const signed char *)Kp.p, (const signed char *)Vp.p, (const float *)Ksc.p,
                         (const float *)Vsc.p, (const float *)Q2.p, P2.as<float>(), n_h, n_kv, hd, scale, softcap, window));
        else
            RC(d->launch(al.f, (unsigned)(items.size() / al.waves), 1, 1, 64 * al.waves, (const void *)I2.p, (const int *)L2.p,
                         (const int *)S2.p, (const int *)T.p, maxBlocks, (const uint16_t *)Kp.p, (const uint16_t *)Vp.p, (const float *)Q2.p, P2.as<float>(), n_h,
                         n_kv, hd, scale, softcap, window));
        RC(d->launch(d->k.attn_combine, (unsigned)n_h, (unsigned)rows, 1, (unsigned)(ATTN_PIECES * hd / 4), (const float *)P2.p, (const int *)St2.p, partRows,
                     O2.as<float>(), n_h, n_kv, hd, (const float *)Sk.p));
        RC(d->d2h(out + (size_t)r0 * qd, O2.p, sizeof(float) * (size_t)rows * qd));
    }
    return RD_OK;
}
extern "C" int rd_attn_ragged(rd_device *d, int n_seq, const int *len, const int64_t *off, const float *k, const float *v, const float *q,
                              int n_h, int n_kv, int hd, float scale, float softcap, float *out) {
    return attn_ragged_typed(d, RD_KV_F16, n_seq, len, nullptr, off, k, v, q, n_h, n_kv, hd, scale, softcap, out);
}
extern "C" int rd_attn_ragged_i8(rd_device *d, int n_seq, const int *len, const int64_t *off, const float *k, const float *v, const float *q,
                                 int n_h, int n_kv, int hd, float scale, float softcap, float *out) {
    return attn_ragged_typed(d, RD_KV_I8, n_seq, len, nullptr, off, k, v, q, n_h, n_kv, hd, scale, softcap, out);
}
extern "C" int rd_attn_ragged_rows(rd_device *d, int kv_type, int n_seq, const int *len, const int *nq, const int64_t *off, const float *k, const float *v,
                                   const float *q, int n_h, int n_kv, int hd, float scale, float softcap, float *out) {
    if (!nq || (kv_type != RD_KV_F16 && kv_type != RD_KV_I8)) return RD_ERR_ARG;
    return attn_ragged_typed(d, kv_type, n_seq, len, nq, off, k, v, q, n_h, n_kv, hd, scale, softcap, out);
}

// The same with a sliding window (each row reads the last `window` positions of its sequence only; 0 = the whole sequence) and
// attention sinks (sinks: host f32 [n_h] or NULL). nq may be NULL (one query row per sequence, the last position).
extern "C" int rd_attn_ragged_ex(rd_device *d, int kv_type, int n_seq, const int *len, const int *nq, const int64_t *off, const float *k, const float *v,
                                 const float *q, int n_h, int n_kv, int hd, float scale, float softcap, int window, const float *sinks, float *out) {
    if ((kv_type != RD_KV_F16 && kv_type != RD_KV_I8) || window < 0) return RD_ERR_ARG;
    return attn_ragged_typed(d, kv_type, n_seq, len, nq, off, k, v, q, n_h, n_kv, hd, scale, softcap, out, window, sinks);
}

// ---- top-K of logits rows (kernel-level entry point) ----
// 1/T as the sampler's device paths take it (backend/cuda/topk.go:74-77): f32(1/T), 1 for T <= 0
static float topk_inv_t(double temperature) { return temperature > 0 ? (float)(1.0 / temperature) : 1.f; }

extern "C" int rd_topk_rows(rd_device *d, const float *logits, int rows, int V, int k, double temperature, int want_z, int *ids, float *vals,
                            double *z) {
    if (!d || !logits || !ids || !vals || (want_z && !z) || rows <= 0 || V <= 0) return RD_ERR_ARG;
    if (k < 1 || k > TOPK_MAX) {
        rd_set_error("rd_topk_rows: k=%d outside [1,%d]", k, TOPK_MAX);
        return RD_ERR_ARG;
    }
    if (k > V) k = V;
    DevBuf L(d), I(d), Vv(d), Z(d);
    RC(L.alloc(sizeof(float) * (size_t)rows * V));
    RC(I.alloc(sizeof(int) * (size_t)rows * k));
    RC(Vv.alloc(sizeof(float) * (size_t)rows * k));
    RC(Z.alloc(sizeof(double) * (size_t)rows));
    RC(d->h2d(L.p, logits, sizeof(float) * (size_t)rows * V));
    TopkScratch sc;
    RC(topk_scratch_alloc(d, rows, V, &sc));
    int rc = launch_topk(d, (const float *)L.p, rows, V, k, topk_inv_t(temperature), false, sc, I.as<int>(), Vv.as<float>(),
                         want_z ? Z.as<double>() : (double *)nullptr);
    if (!rc) rc = d->sync();
    for (void *p : {(void *)sc.ghist, (void *)sc.ccount, (void *)sc.gmax, (void *)sc.cand_i, (void *)sc.cand_v, (void *)sc.invT, (void *)sc.zpart}) d->release(p);
    RC(rc);
    RC(d->d2h(ids, I.p, sizeof(int) * (size_t)rows * k));
    RC(d->d2h(vals, Vv.p, sizeof(float) * (size_t)rows * k));
    if (want_z) RC(d->d2h(z, Z.p, sizeof(double) * (size_t)rows));
    return RD_OK;
}

// ---- the same reduction with nothing allocated: forwards to librocmdecode_static.so ----
// That library (csrc/static/topk_static.hip, built by hipcc) keeps the scratch between the launches in a file-scope device array
// and links the HIP runtime; it sits beside this one and is opened on the first call, so this library itself still binds
// libamdhip64 only at run time.
#include <dlfcn.h>
#include <mutex>
typedef int (*topk_static_fn)(int, void *, const float *, int, int, int, double, int, int *, float *, double *, char *, size_t);
typedef int (*topk_static_prepare_fn)(int, char *, size_t);
struct TopkStaticLib {
    topk_static_fn run = nullptr;
    topk_static_prepare_fn prepare = nullptr;
    std::string err;
};
static const TopkStaticLib &load_topk_static() {
    static std::once_flag once;
    static TopkStaticLib lib;
    std::call_once(once, [] {
        std::string path = "librocmdecode_static.so";
        Dl_info info;
        if (dladdr((void *)&rd_plan_gemm, &info) && info.dli_fname) {
            std::string p = info.dli_fname;
            size_t s = p.find_last_of('/');
            path = (s == std::string::npos ? std::string(".") : p.substr(0, s)) + "/librocmdecode_static.so";
        }
        if (const char *e = getenv("ROCMDECODE_STATIC_LIB")) path = e;
        void *h = dlopen(path.c_str(), RTLD_NOW | RTLD_LOCAL);
        if (!h) {
            lib.err = std::string("cannot load ") + path + ": " + dlerror();
            return;
        }
        lib.run = (topk_static_fn)dlsym(h, "rd_topk_rows_static_impl");
        lib.prepare = (topk_static_prepare_fn)dlsym(h, "rd_topk_static_prepare");
        if (!lib.run || !lib.prepare) lib.run = nullptr, lib.err = path + " lacks rd_topk_rows_static_impl / rd_topk_static_prepare";
    });
    return lib;
}

// rd_device_open's part: the allocation-free library is opened and its scratch address looked up for this device now, so that a
// later rd_topk_rows_static under stream capture has nothing left to set up. A missing library is not this call's error: the entry
// point reports it when it is used.
void topk_static_prepare_device(int ordinal) {
    const TopkStaticLib &lib = load_topk_static();
    if (!lib.run) return;
    char msg[400] = "";
    (void)lib.prepare(ordinal, msg, sizeof msg);
}

extern "C" int rd_topk_rows_static(int device, void *stream, const float *logits_dev, int rows, int V, int k, double temperature, int want_z,
                                   int *ids_dev, float *vals_dev, double *z_dev) {
    const TopkStaticLib &lib = load_topk_static();
    if (!lib.run) {
        rd_set_error("rd_topk_rows_static: %s", lib.err.c_str());
        return RD_ERR_STATE;
    }
    char msg[400] = "";
    int rc = lib.run(device, stream, logits_dev, rows, V, k, temperature, want_z, ids_dev, vals_dev, z_dev, msg, sizeof msg);
    if (rc) rd_set_error("%s", msg);
    return rc;
}

// ---- host planning without a device ----
extern "C" int rd_plan_attention(int rows, const int *len, const int *slot, int heads_per_kv, int n_kv, int *items_out, int max_items, int *ranges_out,
                                 int *n_items, int *grouped) {
    if (rows <= 0 || !len || heads_per_kv <= 0 || n_kv <= 0 || !items_out || !ranges_out || !n_items || !grouped) return RD_ERR_ARG;
    for (int r = 0; r < rows; r++)
        if (len[r] <= 0) {
            rd_set_error("row %d has no keys", r);
            return RD_ERR_ARG;
        }
    std::vector<AttnItemH> items;
    std::vector<int> ranges;
    *grouped = build_attn_worklist(len, slot, heads_per_kv, rows, n_kv, items, ranges) ? 1 : 0;
    *n_items = (int)items.size();
    if ((int)items.size() > max_items) {
        rd_set_error("attention work list of %zu items exceeds %d", items.size(), max_items);
        return RD_ERR_ARG;
    }
    memcpy(items_out, items.data(), sizeof(AttnItemH) * items.size());
    memcpy(ranges_out, ranges.data(), sizeof(int) * ranges.size());
    return RD_OK;
}

extern "C" int rd_plan_gemm(int N, int n_kblocks, int *splits, int *kblocks_per_split) {
    if (N <= 0 || n_kblocks <= 0 || !splits || !kblocks_per_split) return RD_ERR_ARG;
    GemmPlan p = plan_gemm(0, N, n_kblocks);
    *splits = p.splits, *kblocks_per_split = p.kbPerSplit;
    return RD_OK;
}
