/*
 * kprint.c — reproduces goinfer's kernel fingerprints (internal/diag/kernelprint) over the oracle's
 * restatements, so that each restated function is pinned bit for bit without running any Go.
 * TEST INFRASTRUCTURE ONLY (see oracle.h).
 *
 * The recipe is the reference's own (re-implemented, not copied): inputs come from splitmix64 seeded
 * with the little-endian u64 of sha256(kernel name)[:8] (kernelprint.go:86-90, inputs.go:5-15); each call's
 * output bits are hashed after a tag of its shape (kernelprint.go:98-112). The expected digests are the
 * table testdata/kernel_fingerprints.json, carried as data in tests/golden/kernel_fingerprints.json.
 */
#include "oracle.h"
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

/* ---------------- SHA-256 (FIPS 180-4) ---------------- */
typedef struct {
    uint32_t h[8];
    uint8_t buf[64];
    uint64_t len;
    size_t fill;
} sha256;

static const uint32_t KK[64] = {
    0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5, 0xd807aa98, 0x12835b01, 0x243185be,
    0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174, 0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa,
    0x5cb0a9dc, 0x76f988da, 0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967, 0x27b70a85,
    0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85, 0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3,
    0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070, 0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f,
    0x682e6ff3, 0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};
#define ROR(x, n) (((x) >> (n)) | ((x) << (32 - (n))))

static void sha_block(sha256 *s, const uint8_t *p) {
    uint32_t w[64], a, b, c, d, e, f, g, h;
    for (int i = 0; i < 16; i++) w[i] = (uint32_t)p[4 * i] << 24 | (uint32_t)p[4 * i + 1] << 16 | (uint32_t)p[4 * i + 2] << 8 | p[4 * i + 3];
    for (int i = 16; i < 64; i++) {
        uint32_t s0 = ROR(w[i - 15], 7) ^ ROR(w[i - 15], 18) ^ (w[i - 15] >> 3);
        uint32_t s1 = ROR(w[i - 2], 17) ^ ROR(w[i - 2], 19) ^ (w[i - 2] >> 10);
        w[i] = w[i - 16] + s0 + w[i - 7] + s1;
    }
    a = s->h[0], b = s->h[1], c = s->h[2], d = s->h[3], e = s->h[4], f = s->h[5], g = s->h[6], h = s->h[7];
    for (int i = 0; i < 64; i++) {
        uint32_t S1 = ROR(e, 6) ^ ROR(e, 11) ^ ROR(e, 25), ch = (e & f) ^ (~e & g);
        uint32_t t1 = h + S1 + ch + KK[i] + w[i];
        uint32_t S0 = ROR(a, 2) ^ ROR(a, 13) ^ ROR(a, 22), mj = (a & b) ^ (a & c) ^ (b & c);
        uint32_t t2 = S0 + mj;
        h = g, g = f, f = e, e = d + t1, d = c, c = b, b = a, a = t1 + t2;
    }
    s->h[0] += a, s->h[1] += b, s->h[2] += c, s->h[3] += d, s->h[4] += e, s->h[5] += f, s->h[6] += g, s->h[7] += h;
}

static void sha_init(sha256 *s) {
    static const uint32_t iv[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
    memcpy(s->h, iv, sizeof iv);
    s->len = 0;
    s->fill = 0;
}

static void sha_write(sha256 *s, const void *data, size_t n) {
    const uint8_t *p = (const uint8_t *)data;
    s->len += n;
    while (n) {
        size_t take = 64 - s->fill < n ? 64 - s->fill : n;
        memcpy(s->buf + s->fill, p, take);
        s->fill += take, p += take, n -= take;
        if (s->fill == 64) {
            sha_block(s, s->buf);
            s->fill = 0;
        }
    }
}

static void sha_sum(sha256 *s, uint8_t out[32]) {
    uint64_t bits = s->len * 8;
    uint8_t pad = 0x80, z = 0, lenb[8];
    sha_write(s, &pad, 1);
    while (s->fill != 56) sha_write(s, &z, 1);
    for (int i = 0; i < 8; i++) lenb[i] = (uint8_t)(bits >> (56 - 8 * i));
    sha_write(s, lenb, 8);
    for (int i = 0; i < 8; i++) {
        out[4 * i] = (uint8_t)(s->h[i] >> 24), out[4 * i + 1] = (uint8_t)(s->h[i] >> 16);
        out[4 * i + 2] = (uint8_t)(s->h[i] >> 8), out[4 * i + 3] = (uint8_t)s->h[i];
    }
}

/* ---------------- the input generator: internal/diag/kernelprint/inputs.go ---------------- */
typedef struct {
    uint64_t s;
} gen;

static uint64_t g_next(gen *g) {
    g->s += 0x9e3779b97f4a7c15ULL;
    uint64_t z = g->s;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
}
static float g_unit(gen *g) { return (float)((int32_t)(g_next(g) >> 40) - (1 << 23)) * (1.0f / (1 << 23)); }
static float g_bell(gen *g) {
    float a = g_unit(g), b = g_unit(g), c = g_unit(g), d = g_unit(g);
    float s = a + b;
    s = s + c;
    s = s + d;
    return s;
}
static float *g_vec(gen *g, int n, float scale) {
    float *v = (float *)malloc(sizeof(float) * (size_t)(n > 0 ? n : 1));
    for (int i = 0; i < n; i++) {
        float x = g_bell(g) * scale;
        if (i % 13 == 5) x = x * 8;
        v[i] = x;
    }
    return v;
}
static float *g_mat(gen *g, int rows, int cols, float scale) {
    float *m = g_vec(g, rows * cols, scale);
    if (rows > 2) {
        memset(m + cols, 0, sizeof(float) * (size_t)cols);
        float c = g_bell(g) * scale;
        for (int j = 0; j < cols; j++) m[2 * cols + j] = c;
    }
    return m;
}
static float *ties(int cols) {
    float *v = (float *)malloc(sizeof(float) * (size_t)cols);
    for (int j = 0; j < cols; j++) v[j] = (float)(j % 254 - 127) + 0.5f;
    v[0] = 127;
    return v;
}
static uint16_t g_half16_one(gen *g, uint16_t lo, uint16_t hi) {
    uint64_t r = g_next(g);
    uint16_t e = (uint16_t)(lo + (uint16_t)(r % (uint64_t)(hi - lo + 1)));
    return (uint16_t)(((uint16_t)(r >> 8) & 0x8000) | (uint16_t)(e << 10) | ((uint16_t)(r >> 16) & 0x3ff));
}
static uint8_t *g_bytes(gen *g, int n) {
    uint8_t *b = (uint8_t *)malloc((size_t)n + 8);
    for (int i = 0; i < n; i += 8) {
        uint64_t r = g_next(g);
        for (int j = 0; j < 8 && i + j < n; j++) b[i + j] = (uint8_t)(r >> (8 * j));
    }
    return b;
}
/* formats.go:40-53: random blocks with the binary16 fields set to finite values in [2^-10, 2^-3). */
static uint8_t *g_blocks_q4k(gen *g, int n_blocks) {
    uint8_t *raw = g_bytes(g, n_blocks * 144);
    for (int b = 0; b < n_blocks; b++)
        for (int f = 0; f < 2; f++) {
            uint16_t h = g_half16_one(g, 5, 11) & 0x7fff;
            raw[b * 144 + 2 * f] = (uint8_t)h;
            raw[b * 144 + 2 * f + 1] = (uint8_t)(h >> 8);
        }
    return raw;
}
/* the same for any block format: size bytes per block, n16 binary16 fields at the given offsets */
static uint8_t *g_blocks_fmt(gen *g, int n_blocks, int size, const int *f16_at, int n16) {
    uint8_t *raw = g_bytes(g, n_blocks * size);
    for (int b = 0; b < n_blocks; b++)
        for (int f = 0; f < n16; f++) {
            uint16_t h = g_half16_one(g, 5, 11) & 0x7fff;
            raw[b * size + f16_at[f]] = (uint8_t)h;
            raw[b * size + f16_at[f] + 1] = (uint8_t)(h >> 8);
        }
    return raw;
}
static float *g_probs(gen *g, int rows, int nKeys) {
    float *p = (float *)malloc(sizeof(float) * (size_t)rows * nKeys);
    for (int i = 0; i < rows * nKeys; i++) p[i] = (float)(g_unit(g) + 1) * (1.0f / 512);
    return p;
}

/* ---------------- the sink: kernelprint.go:92-131 ---------------- */
static void s_tag(sha256 *s, const char *name, int n, const long *ints) {
    sha_write(s, name, strlen(name));
    for (int i = 0; i < n; i++) {
        uint64_t v = (uint64_t)ints[i];
        uint8_t b[8];
        for (int j = 0; j < 8; j++) b[j] = (uint8_t)(v >> (8 * j));
        sha_write(s, b, 8);
    }
}
static void s_f32(sha256 *s, const float *v, size_t n) { sha_write(s, v, 4 * n); } /* little-endian host */
static void s_u16(sha256 *s, const uint16_t *v, size_t n) { sha_write(s, v, 2 * n); }
static void s_bytes(sha256 *s, const void *v, size_t n) { sha_write(s, v, n); }

static const int mList[] = {1, 2, 3, 4, 5, 8, 9, 16, 17, 33};
static const int kG32[] = {16, 32, 48, 64, 96, 100, 128, 256, 768, 2048};
static const int quantCols[] = {1, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 128, 257, 1000};
static const int headDims[] = {1, 15, 16, 17, 32, 33, 64, 80, 128};
#define LEN(a) ((int)(sizeof(a) / sizeof((a)[0])))

/* probes32: inputs.go:70-84 */
static uint32_t *probes32(int *n_out) {
    static const uint32_t mants[] = {0, 1, 0x0fff, 0x1000, 0x1001, 0x2000, 0x3000, 0x7fff, 0x8000, 0x8001, 0x18000, 0x7fe000, 0x7fefff, 0x7ff000, 0x7fffff};
    uint32_t *out = (uint32_t *)malloc(sizeof(uint32_t) * (71 * 15 * 2 + 6));
    int n = 0;
    for (uint32_t e = 90; e <= 160; e++)
        for (int i = 0; i < 15; i++) {
            out[n++] = e << 23 | mants[i];
            out[n++] = 1u << 31 | e << 23 | mants[i];
        }
    out[n++] = 0, out[n++] = 1u << 31, out[n++] = 0x7f800000, out[n++] = 0xff800000, out[n++] = 1, out[n++] = 0x00400000;
    *n_out = n;
    return out;
}

static void k_f32_to_f16(sha256 *s, gen *g) {
    (void)g;
    int n;
    uint32_t *p = probes32(&n);
    uint16_t *out = (uint16_t *)malloc(2 * (size_t)n);
    for (int i = 0; i < n; i++) {
        float f;
        memcpy(&f, &p[i], 4);
        out[i] = or_f32_to_f16(f);
    }
    s_u16(s, out, (size_t)n);
    free(out);
    free(p);
}

static void k_f16_to_f32(sha256 *s, gen *g) {
    (void)g;
    float *out = (float *)malloc(4 * 65536);
    for (int h = 0; h < 65536; h++) out[h] = or_f16_to_f32((uint16_t)h);
    s_f32(s, out, 65536);
    free(out);
}

/* kernelprint.go:888-918 (ggufTensor1) for Q5_K (ggml type 13) and Q6_K (type 14); formats.go:30-31 give the block shapes */
static void k_gguf_fmt(sha256 *s, gen *g, int size, const int *f16_at, int n16, void (*deq)(const uint8_t *, size_t, float *)) {
    static const int nbs[] = {1, 3}, rws[] = {1, 3};
    for (int a = 0; a < 2; a++)
        for (int b = 0; b < 2; b++) {
            int nb = nbs[a], rows = rws[b], cols = nb * 256, nblk = rows * cols / 256;
            uint8_t *data = g_blocks_fmt(g, nblk, size, f16_at, n16);
            float *out = (float *)malloc(sizeof(float) * (size_t)rows * cols);
            deq(data, (size_t)nblk, out);
            long t[3] = {nb, rows, 2};
            s_tag(s, "t", 3, t);
            s_f32(s, out, (size_t)rows * cols);
            free(out);
            free(data);
        }
}
static void k_gguf_q5k(sha256 *s, gen *g) {
    static const int at[] = {0, 2};
    k_gguf_fmt(s, g, 176, at, 2, or_dequant_q5k);
}
static void k_gguf_q6k(sha256 *s, gen *g) {
    static const int at[] = {208};
    k_gguf_fmt(s, g, 210, at, 1, or_dequant_q6k);
}

/* kernelprint.go:888-918 (ggufTensor1) for Q4_K */
static void k_gguf_q4k(sha256 *s, gen *g) {
    static const int nbs[] = {1, 3}, rws[] = {1, 3};
    for (int a = 0; a < 2; a++)
        for (int b = 0; b < 2; b++) {
            int nb = nbs[a], rows = rws[b], cols = nb * 256, nblk = rows * cols / 256;
            uint8_t *data = g_blocks_q4k(g, nblk);
            float *out = (float *)malloc(sizeof(float) * (size_t)rows * cols);
            or_dequant_q4k(data, (size_t)nblk, out);
            long t[3] = {nb, rows, 2};
            s_tag(s, "t", 3, t);
            s_f32(s, out, (size_t)rows * cols);
            free(out);
            free(data);
        }
}

/* kernelprint.go:344-354 */
static void k_quantize_row_int8(sha256 *s, gen *g) {
    for (int c = 0; c < LEN(quantCols); c++) {
        int cols = quantCols[c];
        float *rows[3] = {g_vec(g, cols, 1), ties(cols), (float *)calloc((size_t)cols, sizeof(float))};
        for (int r = 0; r < 3; r++) {
            int8_t *q = (int8_t *)malloc((size_t)cols);
            float sc = or_quantize_row_int8(rows[r], cols, q);
            long t[1] = {cols};
            s_tag(s, "q", 1, t);
            s_bytes(s, q, (size_t)cols);
            s_f32(s, &sc, 1);
            free(q);
            free(rows[r]);
        }
    }
}

/* kernelprint.go:1005-1016 (int8Rows): rows x cols random codes, then positive per-row scales */
static int8_t *int8_rows(gen *g, int rows, int cols, float **sc_out) {
    int8_t *q = (int8_t *)g_bytes(g, rows * cols);
    float *sc = (float *)malloc(sizeof(float) * (size_t)rows);
    for (int i = 0; i < rows; i++) sc[i] = (float)(g_unit(g) * (1.0 / 64)) + (1.0f / 32);
    *sc_out = sc;
    return q;
}
/* kernelprint.go:366-377 */
static void k_dequantize_rows_int8(sha256 *s, gen *g) {
    static const int rowsList[] = {1, 3, 4};
    for (int ri = 0; ri < 3; ri++)
        for (int c = 0; c < LEN(quantCols); c++) {
            int rows = rowsList[ri], cols = quantCols[c];
            float *sc, *dst = (float *)malloc(sizeof(float) * (size_t)rows * cols);
            int8_t *q = int8_rows(g, rows, cols, &sc);
            or_dequantize_rows_int8(dst, q, sc, rows, cols);
            long t[2] = {rows, cols};
            s_tag(s, "dq", 2, t);
            s_f32(s, dst, (size_t)rows * cols);
            free(q), free(sc), free(dst);
        }
}

/* kernelprint.go:495-515 */
static void k_quantize_act(sha256 *s, gen *g) {
    static const int groups[] = {0, 32}, ks0[] = {1, 7, 17, 33, 100, 256};
    for (int gi = 0; gi < 2; gi++) {
        int group = groups[gi];
        const int *ks = group > 0 ? kG32 : ks0;
        int nk = group > 0 ? LEN(kG32) : LEN(ks0);
        for (int ki = 0; ki < nk; ki++)
            for (int mi = 0; mi < LEN(mList); mi++) {
                int K = ks[ki], M = mList[mi];
                float *a = g_vec(g, M * K, 1);
                if (M > 1) {
                    float *t = ties(K);
                    memcpy(a + K, t, sizeof(float) * (size_t)K);
                    free(t);
                }
                int nG = group > 0 ? (K + group - 1) / group : 1;
                int8_t *q = (int8_t *)malloc((size_t)M * K);
                float *S = (float *)malloc(sizeof(float) * (size_t)M * nG);
                or_quantize_act(a, M, K, group, q, S);
                long t[3] = {group, M, K};
                s_tag(s, "q", 3, t);
                s_bytes(s, q, (size_t)M * K);
                s_f32(s, S, (size_t)M * nG);
                free(q);
                free(S);
                free(a);
            }
    }
}

/* kernelprint.go:472-483 */
static void k_quantize_group_int4_row(sha256 *s, gen *g) {
    static const int groups[] = {32, 64}, colsL[] = {64, 128, 256, 2048};
    for (int gi = 0; gi < 2; gi++)
        for (int ci = 0; ci < 4; ci++) {
            int group = groups[gi], cols = colsL[ci];
            float *rows[3] = {g_vec(g, cols, 1), ties(cols), (float *)calloc((size_t)cols, sizeof(float))};
            for (int r = 0; r < 3; r++) {
                uint8_t *packed = (uint8_t *)malloc((size_t)cols / 2);
                float *sc = (float *)malloc(sizeof(float) * (size_t)(cols / group));
                or_quantize_int4_row(rows[r], cols, group, packed, sc);
                long t[2] = {group, cols};
                s_tag(s, "q", 2, t);
                s_bytes(s, packed, (size_t)cols / 2);
                s_f32(s, sc, (size_t)(cols / group));
                free(packed);
                free(sc);
                free(rows[r]);
            }
        }
}

/* kernelprint.go:484-494 */
static void k_quantize_int4(sha256 *s, gen *g) {
    static const int rc[4][2] = {{1, 32}, {3, 64}, {4, 256}, {8, 2048}};
    for (int i = 0; i < 4; i++) {
        int rows = rc[i][0], cols = rc[i][1], nG = cols / 32;
        float *w = g_mat(g, rows, cols, 1);
        uint8_t *q4 = (uint8_t *)malloc((size_t)rows * cols / 2);
        uint16_t *s16 = (uint16_t *)malloc(2 * (size_t)rows * nG);
        or_quantize_int4_mat(w, rows, cols, 32, q4, s16);
        long t[3] = {rows, cols, 32};
        s_tag(s, "q", 3, t);
        uint8_t one = 1;
        s_bytes(s, &one, 1);
        s_bytes(s, q4, (size_t)rows * cols / 2);
        s_u16(s, s16, (size_t)rows * nG);
        free(w);
        free(q4);
        free(s16);
    }
}

/* kernelprint.go:673-686 and 701-715 */
static void k_qk_acc64(sha256 *s, gen *g) {
    static const int nk[] = {1, 2, 7, 64, 513}, ms[] = {1, 2, 5, 17};
    for (int hi = 0; hi < LEN(headDims); hi++)
        for (int ki = 0; ki < 5; ki++)
            for (int mi = 0; mi < 4; mi++) {
                int hd = headDims[hi], nKeys = nk[ki], M = ms[mi], kvDim = 2 * hd + 3;
                float *a = g_vec(g, M * hd, 1), *keys = g_vec(g, nKeys * kvDim, 1);
                float *dst = (float *)malloc(sizeof(float) * (size_t)M * nKeys);
                or_qk_acc64(a, keys, dst, M, hd, nKeys, hd, kvDim);
                long t[3] = {hd, nKeys, M};
                s_tag(s, "qk", 3, t);
                s_f32(s, dst, (size_t)M * nKeys);
                free(a);
                free(keys);
                free(dst);
            }
}

static void k_av_acc64(sha256 *s, gen *g) {
    static const int nk[] = {1, 2, 7, 64, 513}, ms[] = {1, 2, 5, 17};
    for (int hi = 0; hi < LEN(headDims); hi++)
        for (int ki = 0; ki < 5; ki++)
            for (int mi = 0; mi < 4; mi++) {
                int hd = headDims[hi], nKeys = nk[ki], M = ms[mi], kvDim = 2 * hd + 3;
                float *sc = g_probs(g, M, nKeys), *vals = g_vec(g, nKeys * kvDim, 1);
                float *dst = (float *)malloc(sizeof(float) * (size_t)M * hd);
                or_av_acc64(sc, vals, dst, M, nKeys, hd, hd, kvDim);
                long t[3] = {hd, nKeys, M};
                s_tag(s, "av", 3, t);
                s_f32(s, dst, (size_t)M * hd);
                free(sc);
                free(vals);
                free(dst);
            }
}

static const int mLarge[] = {1, 2, 5, 17}, nLarge[] = {1, 4, 9, 33};
static const int nList[] = {1, 2, 3, 4, 5, 7, 8, 9, 16, 17, 33};
static const int kQ8[] = {1, 7, 16, 17, 32, 33, 64, 100, 128, 256, 768, 2048};
static const int thresholds[] = {-1, 1, 300000, 1 << 20};

/* one W8A8 shape: a = vec(M*K,1); weights = QuantizeRowsInt8(mat(N,K,0.25)) (kernelprint.go:405-418) */
static void w8a8_shape(sha256 *s, gen *g, int M, int K, int N, int group, const long *tag, int ntag) {
    float *a = g_vec(g, M * K, 1), *w = g_mat(g, N, K, 0.25f);
    int8_t *q = (int8_t *)malloc((size_t)N * K);
    float *sc = (float *)malloc(sizeof(float) * (size_t)N), *dst = (float *)malloc(sizeof(float) * (size_t)M * N);
    for (int n = 0; n < N; n++) sc[n] = or_quantize_row_int8(w + (size_t)n * K, K, q + (size_t)n * K);
    or_mat wm = {OR_W8A8, N, K, q, sc, group};
    or_matmul(&wm, a, M, dst);
    s_tag(s, "mm", ntag, tag);
    s_f32(s, dst, (size_t)M * N);
    free(a), free(w), free(q), free(sc), free(dst);
}

/* kernelprint.go:157-170 (shapes): fewer M and N at K >= 768 */
static void w8a8_shapes(sha256 *s, gen *g, const int *ks, int nks, int group, int thr, int with_prefix) {
    for (int ki = 0; ki < nks; ki++) {
        int K = ks[ki];
        const int *ms = mList, *ns = nList;
        int nm = LEN(mList), nn = LEN(nList);
        if (K >= 768) ms = mLarge, ns = nLarge, nm = 4, nn = 4;
        for (int mi = 0; mi < nm; mi++)
            for (int ni = 0; ni < nn; ni++) {
                long t5[5] = {group, thr, ms[mi], K, ns[ni]};
                if (with_prefix)
                    w8a8_shape(s, g, ms[mi], K, ns[ni], group, t5, 5);
                else
                    w8a8_shape(s, g, ms[mi], K, ns[ni], group, t5 + 2, 3);
            }
    }
}

/* kernelprint.go:439-448: per-row activations, every configuration agrees on this digest */
static void k_matmul_w8a8(sha256 *s, gen *g) { w8a8_shapes(s, g, kQ8, LEN(kQ8), 0, 0, 0); }

/* kernelprint.go:421-438: per-row then per-32 activations, over the four fan-out thresholds (which change no bits) */
static void k_matmul_w8a8_into(sha256 *s, gen *g) {
    for (int gi = 0; gi < 2; gi++)
        for (int ti = 0; ti < 4; ti++)
            w8a8_shapes(s, g, gi ? kG32 : kQ8, gi ? LEN(kG32) : LEN(kQ8), gi ? 32 : 0, thresholds[ti], 1);
}

typedef struct {
    const char *name;
    void (*run)(sha256 *, gen *);
} kernel;

static const kernel suite[] = {
    {"linalg.F32ToF16", k_f32_to_f16},
    {"linalg.F16ToF32", k_f16_to_f32},
    {"embed.GGUFFile(Q4_K).Tensor", k_gguf_q4k},
    {"embed.GGUFFile(Q5_K).Tensor", k_gguf_q5k},
    {"embed.GGUFFile(Q6_K).Tensor", k_gguf_q6k},
    {"linalg.QuantizeRowInt8", k_quantize_row_int8},
    {"linalg.DequantizeRowsInt8Into", k_dequantize_rows_int8},
    {"linalg.QuantizeActQ", k_quantize_act},
    {"linalg.QuantizeGroupInt4Row", k_quantize_group_int4_row},
    {"linalg.QuantizeInt4", k_quantize_int4},
    {"linalg.MatmulQKAcc64", k_qk_acc64},
    {"linalg.MatmulAVAcc64", k_av_acc64},
    {"linalg.MatmulBTW8A8", k_matmul_w8a8},
    {"linalg.MatmulBTW8A8Into", k_matmul_w8a8_into},
};

int or_kprint_count(void) { return LEN(suite); }
const char *or_kprint_name(int i) { return (i >= 0 && i < LEN(suite)) ? suite[i].name : NULL; }

/* Writes "sha256:<hex>" (71 chars + NUL) for suite entry i; returns 0 on success. */
int or_kprint_run(int i, char out[80]) {
    if (i < 0 || i >= LEN(suite)) return -1;
    uint8_t d[32];
    sha256 seed_h, s;
    sha_init(&seed_h);
    sha_write(&seed_h, suite[i].name, strlen(suite[i].name));
    sha_sum(&seed_h, d);
    gen g = {0};
    for (int j = 0; j < 8; j++) g.s |= (uint64_t)d[j] << (8 * j);
    sha_init(&s);
    suite[i].run(&s, &g);
    sha_sum(&s, d);
    strcpy(out, "sha256:");
    for (int j = 0; j < 32; j++) sprintf(out + 7 + 2 * j, "%02x", d[j]);
    return 0;
}

#ifdef KPRINT_MAIN
int main(void) {
    char out[80];
    for (int i = 0; i < LEN(suite); i++) {
        or_kprint_run(i, out);
        printf("%s %s\n", suite[i].name, out);
    }
    return 0;
}
#endif
