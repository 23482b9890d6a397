// synth.cc — deterministic synthetic weights and activations for tests and benchmarks (libgoinfer_synth.so).
// goinfer has no f32 -> Q4_K quantizer (its fixtures are random valid blocks, decoder/q4k_test.go:14-31), so the
// "N(0, sigma) quantized to Q4_K" inputs of the benchmark configurations are produced here with a ggml-style
// min/max quantizer; parity is defined on the bytes, which the GPU path and the CPU oracle both consume.
// Values are counter-based (a hash of seed and element index), so any slice can be generated independently and in parallel.
#include <math.h>
#include <stdint.h>
#include <string.h>
#include <vector>

static inline uint64_t mix64(uint64_t z) {
    z += 0x9e3779b97f4a7c15ULL;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
}

// Irwin-Hall(12) normal approximation from three 64-bit hashes: exact integer arithmetic, unit variance.
static inline float normal_at(uint64_t seed, uint64_t i) {
    uint64_t k = mix64(seed) ^ (i * 3);
    int32_t s = 0;
    for (int j = 0; j < 3; j++) {
        uint64_t h = mix64(k + (uint64_t)j);
        s += (int32_t)(h & 0xffff) + (int32_t)((h >> 16) & 0xffff) + (int32_t)((h >> 32) & 0xffff) + (int32_t)(h >> 48);
    }
    return (float)(s - 393210) * (1.0f / 65536.0f);
}

static inline float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000) << 16, exp = (h >> 10) & 0x1F, man = h & 0x3FF, u;
    float f;
    if (exp == 0) {
        f = (float)man * 5.9604644775390625e-08f; /* man * 2^-24 */
        return sign ? -f : f;
    }
    u = exp == 0x1F ? (sign | 0x7F800000u | (man << 13)) : (sign | ((exp + 112) << 23) | (man << 13));
    memcpy(&f, &u, 4);
    return f;
}
// round-to-nearest-even binary16 of a finite, non-negative, in-range value (the block scales d and dmin)
static inline uint16_t f32_to_f16_rne(float f) {
    if (!(f > 0.f)) return 0;
    if (f >= 65504.f) return 0x7BFF;
    int e;
    float m = frexpf(f, &e); // f = m * 2^e, m in [0.5,1)
    int be = e - 1 + 15;     // biased exponent of the normal form 1.x * 2^(e-1)
    if (be <= 0) {           // subnormal: units of 2^-24
        float q = nearbyintf(f * 16777216.0f);
        return (uint16_t)q;
    }
    float q = nearbyintf(m * 2048.0f); // 11 significant bits, in [1024, 2048]
    if (q >= 2048.0f) {
        q = 1024.0f;
        be++;
    }
    return (uint16_t)((be << 10) | ((int)q - 1024));
}
// round-half-up binary16, the reference's scale narrowing (internal/runtime/f16/f16.go:14-43)
static inline uint16_t f32_to_f16_half_up(float f) {
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

extern "C" void synth_normal(uint64_t seed, uint64_t offset, size_t n, float mean, float sigma, float *out) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < n; i++) out[i] = mean + sigma * normal_at(seed, offset + i);
}

// One super-block: 256 f32 -> 144 bytes (ggml layout).
static void quantize_block_q4k(const float *x, uint8_t *blk) {
    float scales[8], mins[8];
    float max_scale = 0.f, max_min = 0.f;
    for (int j = 0; j < 8; j++) {
        float mn = x[j * 32], mx = x[j * 32];
        for (int l = 1; l < 32; l++) {
            float v = x[j * 32 + l];
            if (v < mn) mn = v;
            if (v > mx) mx = v;
        }
        if (mn > 0.f) mn = 0.f;
        scales[j] = (mx - mn) / 15.f;
        mins[j] = -mn;
        if (scales[j] > max_scale) max_scale = scales[j];
        if (mins[j] > max_min) max_min = mins[j];
    }
    uint16_t dh = f32_to_f16_rne(max_scale / 63.f), mh = f32_to_f16_rne(max_min / 63.f);
    float d = f16_to_f32(dh), dmin = f16_to_f32(mh);
    uint8_t ls[8], lm[8];
    for (int j = 0; j < 8; j++) {
        int s = d > 0.f ? (int)lrintf(scales[j] / d) : 0, m = dmin > 0.f ? (int)lrintf(mins[j] / dmin) : 0;
        ls[j] = (uint8_t)(s < 0 ? 0 : (s > 63 ? 63 : s));
        lm[j] = (uint8_t)(m < 0 ? 0 : (m > 63 ? 63 : m));
    }
    blk[0] = (uint8_t)dh, blk[1] = (uint8_t)(dh >> 8), blk[2] = (uint8_t)mh, blk[3] = (uint8_t)(mh >> 8);
    uint8_t *q = blk + 4;
    memset(q, 0, 12);
    for (int j = 0; j < 8; j++) {
        if (j < 4) {
            q[j] |= ls[j];
            q[j + 4] |= lm[j];
        } else {
            q[j + 4] = (uint8_t)((ls[j] & 0xF) | ((lm[j] & 0xF) << 4));
            q[j - 4] |= (uint8_t)((ls[j] >> 4) << 6);
            q[j] |= (uint8_t)((lm[j] >> 4) << 6);
        }
    }
    uint8_t *qs = blk + 16;
    memset(qs, 0, 128);
    for (int j = 0; j < 8; j++) {
        float dl = d * (float)ls[j], ml = dmin * (float)lm[j];
        for (int l = 0; l < 32; l++) {
            int v = dl > 0.f ? (int)lrintf((x[j * 32 + l] + ml) / dl) : 0;
            v = v < 0 ? 0 : (v > 15 ? 15 : v);
            qs[(j / 2) * 32 + l] |= (uint8_t)(v << (4 * (j & 1)));
        }
    }
}

extern "C" void synth_quantize_q4k(const float *w, int N, int K, uint8_t *blocks) {
    size_t nb = (size_t)N * (K / 256);
#pragma omp parallel for schedule(static)
    for (size_t b = 0; b < nb; b++) quantize_block_q4k(w + b * 256, blocks + b * 144);
}

// N x K weights ~ N(0, sigma), element (n,k) = normal_at(seed, n*K+k), quantized to Q4_K without materializing the f32 matrix.
extern "C" void synth_q4k_normal(uint64_t seed, int N, int K, float sigma, uint8_t *blocks) {
    size_t nb = (size_t)N * (K / 256);
#pragma omp parallel for schedule(static)
    for (size_t b = 0; b < nb; b++) {
        float x[256];
        for (int i = 0; i < 256; i++) x[i] = sigma * normal_at(seed, b * 256 + i);
        quantize_block_q4k(x, blocks + b * 144);
    }
}

// One super-block: 256 f32 -> 176 bytes of Q5_K (ggml layout): the Q4_K header, 32 levels per sub-block.
static void quantize_block_q5k(const float *x, uint8_t *blk) {
    float scales[8], mins[8];
    float max_scale = 0.f, max_min = 0.f;
    for (int j = 0; j < 8; j++) {
        float mn = x[j * 32], mx = x[j * 32];
        for (int l = 1; l < 32; l++) {
            float v = x[j * 32 + l];
            if (v < mn) mn = v;
            if (v > mx) mx = v;
        }
        if (mn > 0.f) mn = 0.f;
        scales[j] = (mx - mn) / 31.f;
        mins[j] = -mn;
        if (scales[j] > max_scale) max_scale = scales[j];
        if (mins[j] > max_min) max_min = mins[j];
    }
    uint16_t dh = f32_to_f16_rne(max_scale / 63.f), mh = f32_to_f16_rne(max_min / 63.f);
    float d = f16_to_f32(dh), dmin = f16_to_f32(mh);
    uint8_t ls[8], lm[8];
    for (int j = 0; j < 8; j++) {
        int s = d > 0.f ? (int)lrintf(scales[j] / d) : 0, m = dmin > 0.f ? (int)lrintf(mins[j] / dmin) : 0;
        ls[j] = (uint8_t)(s < 0 ? 0 : (s > 63 ? 63 : s));
        lm[j] = (uint8_t)(m < 0 ? 0 : (m > 63 ? 63 : m));
    }
    memset(blk, 0, 176);
    blk[0] = (uint8_t)dh, blk[1] = (uint8_t)(dh >> 8), blk[2] = (uint8_t)mh, blk[3] = (uint8_t)(mh >> 8);
    uint8_t *q = blk + 4;
    for (int j = 0; j < 8; j++) {
        if (j < 4) {
            q[j] |= ls[j];
            q[j + 4] |= lm[j];
        } else {
            q[j + 4] = (uint8_t)((ls[j] & 0xF) | ((lm[j] & 0xF) << 4));
            q[j - 4] |= (uint8_t)((ls[j] >> 4) << 6);
            q[j] |= (uint8_t)((lm[j] >> 4) << 6);
        }
    }
    uint8_t *qh = blk + 16, *qs = blk + 48;
    for (int j = 0; j < 8; j++) {
        float dl = d * (float)ls[j], ml = dmin * (float)lm[j];
        for (int l = 0; l < 32; l++) {
            int v = dl > 0.f ? (int)lrintf((x[j * 32 + l] + ml) / dl) : 0;
            v = v < 0 ? 0 : (v > 31 ? 31 : v);
            qs[(j / 2) * 32 + l] |= (uint8_t)((v & 15) << (4 * (j & 1)));
            qh[l] |= (uint8_t)((v >> 4) << j);
        }
    }
}

// One super-block: 256 f32 -> 210 bytes of Q6_K (ggml layout): 16 sub-blocks of 16, symmetric codes in [-32, 31].
static void quantize_block_q6k(const float *x, uint8_t *blk) {
    float scales[16], max_abs_scale = 0.f;
    for (int j = 0; j < 16; j++) {
        float am = 0.f, sv = 0.f;
        for (int l = 0; l < 16; l++) {
            float v = x[j * 16 + l];
            if (fabsf(v) > am) am = fabsf(v), sv = v;
        }
        scales[j] = -sv / 32.f; // the largest magnitude lands on code -32, as ggml's make_qx_quants does
        if (fabsf(scales[j]) > max_abs_scale) max_abs_scale = fabsf(scales[j]);
    }
    memset(blk, 0, 210);
    uint16_t dh = f32_to_f16_rne(max_abs_scale / 127.f);
    float d = f16_to_f32(dh);
    blk[208] = (uint8_t)dh, blk[209] = (uint8_t)(dh >> 8);
    for (int j = 0; j < 16; j++) {
        int s = d > 0.f ? (int)lrintf(scales[j] / d) : 0;
        s = s < -128 ? -128 : (s > 127 ? 127 : s);
        blk[192 + j] = (uint8_t)(int8_t)s;
    }
    for (int e = 0; e < 256; e++) {
        int half = e / 128, r = e % 128, g = r / 32, l = r % 32;
        float dl = d * (float)(int8_t)blk[192 + e / 16];
        int v = dl != 0.f ? (int)lrintf(x[e] / dl) : 0;
        v = (v < -32 ? -32 : (v > 31 ? 31 : v)) + 32;
        blk[64 * half + 32 * (g & 1) + l] |= (uint8_t)((v & 15) << (4 * (g >> 1)));
        blk[128 + 32 * half + l] |= (uint8_t)((v >> 4) << (2 * g));
    }
}

// N x K weights ~ N(0, sigma), element (n,k) = normal_at(seed, n*K+k), as Q5_K (fmt 5) or Q6_K (fmt 6) super-blocks.
extern "C" void synth_kquant_normal(int fmt, uint64_t seed, int N, int K, float sigma, uint8_t *blocks) {
    size_t nb = (size_t)N * (K / 256);
#pragma omp parallel for schedule(static)
    for (size_t b = 0; b < nb; b++) {
        float x[256];
        for (int i = 0; i < 256; i++) x[i] = sigma * normal_at(seed, b * 256 + i);
        if (fmt == 5)
            quantize_block_q5k(x, blocks + b * 176);
        else
            quantize_block_q6k(x, blocks + b * 210);
    }
}

// int8 rows with the reference's rule (aikit QuantizeRowInt8: scale maxabs/127, round half away, zero row -> scale 1).
extern "C" void synth_w8a8_normal(uint64_t seed, int N, int K, float sigma, int8_t *q, float *scales) {
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; n++) {
        std::vector<float> x((size_t)K);
        float ma = 0.f;
        for (int k = 0; k < K; k++) {
            x[k] = sigma * normal_at(seed, (uint64_t)n * K + k);
            ma = fmaxf(ma, fabsf(x[k]));
        }
        float sc = ma > 0.f ? ma / 127.f : 1.f, inv = ma > 0.f ? 1.f / sc : 0.f;
        for (int k = 0; k < K; k++) {
            float r = roundf(x[k] * inv);
            r = r > 127.f ? 127.f : (r < -127.f ? -127.f : r);
            q[(size_t)n * K + k] = (int8_t)(int)r;
        }
        scales[n] = sc;
    }
}

// int4 group-32 with the reference's rule (decoder/fakequant.go:52-56: scale maxabs/7, codes [-7,7] round half away,
// binary16 scale rounded half up; canonical nibble order, value nib-8).
extern "C" void synth_w4a8_normal(uint64_t seed, int N, int K, float sigma, uint8_t *nib, uint16_t *s16) {
    int nG = K / 32;
#pragma omp parallel for schedule(static)
    for (int n = 0; n < N; n++) {
        uint8_t *row = nib + (size_t)n * (K / 2);
        memset(row, 0, (size_t)K / 2);
        for (int g = 0; g < nG; g++) {
            float x[32], mx = 0.f;
            for (int i = 0; i < 32; i++) {
                x[i] = sigma * normal_at(seed, (uint64_t)n * K + g * 32 + i);
                mx = fmaxf(mx, fabsf(x[i]));
            }
            float s = mx > 0.f ? mx / 7.f : 1.f, inv = 1.f / s;
            s16[(size_t)n * nG + g] = f32_to_f16_half_up(s);
            for (int i = 0; i < 32; i++) {
                float c = roundf(x[i] * inv);
                c = c > 7.f ? 7.f : (c < -7.f ? -7.f : c);
                int k = g * 32 + i;
                row[k >> 1] |= (uint8_t)(((int)c + 8) << (4 * (k & 1)));
            }
        }
    }
}
