// attn.h — paged f16 KV cache and ragged flash-decode attention (goinfer decoder/forwardn.go:295-500 semantics; the CUDA
// analogue is backend/cuda/decode_fa.cu + kvpage.cuh). One query position per sequence, every sequence its own length.
//
// KV pool, per layer: [block][kv head] regions of 64 positions. Inside a region the elements are stored in the order the
// MFMA operand fragments are read, so every wave load is one contiguous 1 KB read:
//   K region: [key tile of 16 (4)][d step c (HD/32)][lane = dq*16 + key][8 halves],   d = dq*(HD/4) + c*8 + i
//   V region: [key tile of 32 (2)][d column tile ct (HD/16)][lane = kq*16 + dcol][8 halves], key = kq*8 + i, d = ct*16 + dcol
// Values are binary16 narrowed with round-half-up, as goinfer's f16 KV cache narrows them (decoder/kvcache.go:21-40).
//
// The int8 cache (goinfer's kvI8: decoder/kvcache.go:43-52 quantizeHeads, backend/cuda/kv8_store.cu, kvtype.cuh:48-73) holds per
// (position, kv head) HD codes and one f32 scale for K and one for V: scale = maxabs/127, code = round-half-away(x/scale)
// clamped to +-127, an all-zero head scale 1; a reader takes code * scale. The pool stores code + 128 as an unsigned byte. Its regions are the same fragment orders in bytes,
// two 8-byte fragments per 16-byte lane slot so that a wave load stays 1 KB:
//   K region: [key tile of 16 (4)][d step pair (HD/64)][lane = dq*16 + key][2 x 8 bytes]   (steps 2cp, 2cp+1)
//   V region: [key tile of 32 (2)][d column tile pair (HD/32)][lane = kq*16 + dcol][2 x 8 bytes]   (tiles 2cp, 2cp+1)
// and the scales sit beside them as [block][kv head][64 positions] f32.
#pragma once
#include "common.h"

template <int HD> __device__ __forceinline__ int k_elem_index(int p, int d) {
    int kt = p >> 4, key = p & 15, dq = d / (HD / 4), rem = d % (HD / 4), c = rem >> 3, i = rem & 7;
    return (((kt * (HD / 32) + c) * 64 + dq * 16 + key) << 3) + i;
}
template <int HD> __device__ __forceinline__ int v_elem_index(int p, int d) {
    int kt = p >> 5, pk = p & 31, kq = pk >> 3, i = pk & 7, ct = d >> 4, dcol = d & 15;
    return (((kt * (HD / 16) + ct) * 64 + kq * 16 + dcol) << 3) + i;
}

template <int HD> __device__ __forceinline__ int k8_elem_index(int p, int d) {
    int kt = p >> 4, key = p & 15, dq = d / (HD / 4), rem = d % (HD / 4), c = rem >> 3, i = rem & 7;
    return (((kt * (HD / 64) + (c >> 1)) * 64 + dq * 16 + key) << 4) + (c & 1) * 8 + i;
}
template <int HD> __device__ __forceinline__ int v8_elem_index(int p, int d) {
    int kt = p >> 5, pk = p & 31, kq = pk >> 3, i = pk & 7, ct = d >> 4, dcol = d & 15;
    return (((kt * (HD / 32) + (ct >> 1)) * 64 + kq * 16 + dcol) << 4) + (ct & 1) * 8 + i;
}
__device__ __forceinline__ int k8_index(int HD, int p, int d) { return HD == 128 ? k8_elem_index<128>(p, d) : k8_elem_index<64>(p, d); }
__device__ __forceinline__ int v8_index(int HD, int p, int d) { return HD == 128 ? v8_elem_index<128>(p, d) : v8_elem_index<64>(p, d); }

// linalg.QuantizeRowInt8's rule for one value, given the head's scale (backend/cuda/kv8_store.cu:27-35)
// The pool keeps code + 128 as an unsigned byte: under a 0x64 high byte that is the f16 value 1024 + 128 + code with no further work.
__device__ __forceinline__ unsigned char kv8_code(float x, float inv) {
    float r = roundf(__fmul_rn(x, inv)); // round half away from zero
    r = fminf(127.f, fmaxf(-127.f, r));
    return (unsigned char)((int)r + 128);
}
// scale and its reciprocal from the head's largest magnitude: maxabs/127, or 1 for an all-zero head (then every code is 0)
__device__ __forceinline__ float kv8_scale(float maxabs, float *inv) {
    float sc = 1.f;
    *inv = 0.f;
    if (maxabs != 0.f) sc = __fdiv_rn(maxabs, 127.f), *inv = __fdiv_rn(1.f, sc);
    return sc;
}

// Host-provided rows into the int8 cache: grid (n, nKV), block 64; lane l quantizes elements l, l+64 of the head.
extern "C" __global__ __launch_bounds__(64) void rd_k_kv_store_i8(const float *__restrict__ k, const float *__restrict__ v, signed char *__restrict__ Kp,
                                                                  signed char *__restrict__ Vp, float *__restrict__ Ksc, float *__restrict__ Vsc,
                                                                  const int *__restrict__ table, int base, int nKV, int HD) {
    const int i = blockIdx.x, kvh = blockIdx.y, lane = threadIdx.x;
    const int pos = base + i, blk = table[pos >> 6], p = pos & 63;
    const size_t region = ((size_t)blk * nKV + kvh) * 64 * HD, srow = ((size_t)blk * nKV + kvh) * 64 + p;
    for (int which = 0; which < 2; which++) {
        const float *src = (which ? v : k) + (size_t)i * nKV * HD + (size_t)kvh * HD;
        float x0 = lane < HD ? src[lane] : 0.f, x1 = lane + 64 < HD ? src[lane + 64] : 0.f;
        float ma = fmaxf(fabsf(x0), fabsf(x1));
        for (int o = 32; o > 0; o >>= 1) ma = fmaxf(ma, __shfl_xor(ma, o, 64));
        float inv, sc = kv8_scale(ma, &inv);
        unsigned char *dst = (unsigned char *)(which ? Vp : Kp) + region;
        if (lane < HD) dst[which ? v8_index(HD, p, lane) : k8_index(HD, p, lane)] = kv8_code(x0, inv);
        if (lane + 64 < HD) dst[which ? v8_index(HD, p, lane + 64) : k8_index(HD, p, lane + 64)] = kv8_code(x1, inv);
        if (lane == 0) (which ? Vsc : Ksc)[srow] = sc;
    }
}

__device__ __forceinline__ void kv_store_elem(uint16_t *__restrict__ Kp, uint16_t *__restrict__ Vp, int HD, size_t region, int p, int d, float kv,
                                              float vv) {
    int ki = HD == 128 ? k_elem_index<128>(p, d) : k_elem_index<64>(p, d);
    int vi = HD == 128 ? v_elem_index<128>(p, d) : v_elem_index<64>(p, d);
    Kp[region + ki] = f32_to_f16_half_up(kv);
    Vp[region + vi] = f32_to_f16_half_up(vv);
}

// Host-provided rows (UploadKV, decoder/resident/forward.go:20-26): k,v f32 [n][nKV*HD] -> positions base..base+n-1 of one sequence.
// Grid (n, nKV), block HD threads: one block per (position, kv head), whatever the number of kv heads.
extern "C" __global__ void rd_k_kv_store(const float *__restrict__ k, const float *__restrict__ v, uint16_t *__restrict__ Kp,
                                         uint16_t *__restrict__ Vp, const int *__restrict__ table, int base, int nKV, int HD) {
    int i = blockIdx.x, kvh = blockIdx.y, d = threadIdx.x;
    if (d >= HD) return;
    int pos = base + i, blk = table[pos >> 6], p = pos & 63;
    size_t region = ((size_t)blk * nKV + kvh) * 64 * HD, src = ((size_t)i * nKV + kvh) * HD + d;
    kv_store_elem(Kp, Vp, HD, region, p, d, k[src], v[src]);
}

// Rows back out of the cache, widened to f32 exactly as an attention read sees them (the host copy a KV snapshot takes,
// decoder/resident/subsystems.go:280-287 SnapshotKV): positions base..base+n-1 of one sequence into k,v f32 [n][nKV*HD].
// f16 cache: the stored binary16 widened; int8 cache: code * scale (linalg.DequantizeRowsInt8Into). Grid (n, nKV), block HD.
extern "C" __global__ void rd_k_kv_read(const void *__restrict__ KpV, const void *__restrict__ VpV, const float *__restrict__ Ksc,
                                        const float *__restrict__ Vsc, float *__restrict__ k, float *__restrict__ v, const int *__restrict__ table,
                                        int base, int nKV, int HD, int i8) {
    int i = blockIdx.x, kvh = blockIdx.y, d = threadIdx.x;
    if (d >= HD) return;
    int pos = base + i, blk = table[pos >> 6], p = pos & 63;
    size_t region = ((size_t)blk * nKV + kvh) * 64 * HD, dst = ((size_t)i * nKV + kvh) * HD + d;
    if (i8) {
        size_t srow = ((size_t)blk * nKV + kvh) * 64 + p;
        int kc = (int)((const unsigned char *)KpV)[region + k8_index(HD, p, d)] - 128, vc = (int)((const unsigned char *)VpV)[region + v8_index(HD, p, d)] - 128;
        k[dst] = __fmul_rn((float)kc, Ksc[srow]);
        v[dst] = __fmul_rn((float)vc, Vsc[srow]);
    } else {
        int ki = HD == 128 ? k_elem_index<128>(p, d) : k_elem_index<64>(p, d);
        int vi = HD == 128 ? v_elem_index<128>(p, d) : v_elem_index<64>(p, d);
        k[dst] = f16_bits_to_f32(((const uint16_t *)KpV)[region + ki]);
        v[dst] = f16_bits_to_f32(((const uint16_t *)VpV)[region + vi]);
    }
}

// NeoX rotation of the pair (x1, x2) = elements (d, d + HD/2) by the angle whose cosine and sine are c, s: products and sum
// each rounded once in f64, then one rounding to f32 (decoder/rope.go:28-64 as amd64 computes it, without fused multiply-adds).
__device__ __forceinline__ float rope_first(float x1, float x2, double c, double s) { return (float)__dsub_rn(__dmul_rn((double)x1, c), __dmul_rn((double)x2, s)); }
__device__ __forceinline__ float rope_second(float x1, float x2, double c, double s) { return (float)__dadd_rn(__dmul_rn((double)x2, c), __dmul_rn((double)x1, s)); }

// The resident model stores the rows of its q|k|v weight so that a rotation pair (d, d + HD/2) of a head falls into one 32-row
// GEMM tile: tile j of a head holds d = 16j .. 16j+15 in its first sixteen rows and d + HD/2 in the other sixteen. Column of
// element d of a head in that order:
__device__ __forceinline__ int qkv_col(int d, int HD) {
    const int half = HD >> 1, dd = d >= half ? d - half : d;
    return ((dd >> 4) << 5) + (dd & 15) + (d >= half ? 16 : 0);
}

// cos and sin of every row's RoPE angles, once per step for all layers (the angle depends on the position and the pair only):
// cs[row][t] = (cos, sin)(pos[row] * invFreq[t]) in f64. Grid (rows), block HD/2.
extern "C" __global__ void rd_k_rope_table(const int *__restrict__ rowPos, const double *__restrict__ invFreq, double2 *__restrict__ cs, int half) {
    const int m = blockIdx.x, t = threadIdx.x;
    if (t >= half) return;
    const double theta = __dmul_rn((double)rowPos[m], invFreq[t]);
    cs[(size_t)m * half + t] = make_double2(cos(theta), sin(theta));
}

// After the q|k|v GEMM: reduce its split-K partials, optional q|k|v bias (Qwen2; decoder/attention.go:12-34 addBias, applied right
// after the projections, program_cpu_n.go:470-476), optional per-head RMSNorm of q and k (Qwen3, decoder/program_cpu.go:351-364),
// NeoX RoPE with f64 angles (decoder/rope.go:28-64), q -> f32 buffer, k,v -> this position of the row's sequence in the pool.
// Grid (nH + 2*nKV, rows), block HD/2 threads... one thread per rotation pair.  P: [splits][32][(nH+2nKV)*HD].
// permuted: the columns of a head in P are in the resident model's q|k|v row order (qkv_col).
template <bool I8>
__device__ __forceinline__ void qkv_rope_store_body(const float *__restrict__ P, int splits, float *__restrict__ q, void *__restrict__ KpV,
                                               void *__restrict__ VpV, float *__restrict__ Ksc, float *__restrict__ Vsc,
                                               const int *__restrict__ tables, int tabStride,
                                               const int *__restrict__ rowSlot, const int *__restrict__ rowPos, const double *__restrict__ invFreq,
                                               const float *__restrict__ qnorm, const float *__restrict__ knorm, float eps, int nH, int nKV, int HD,
                                               size_t pStride, const float *__restrict__ bias, int permuted) {
    int head = blockIdx.x, m = blockIdx.y, t = threadIdx.x, half = HD / 2; // one wave: half <= 64
    const int c1 = permuted ? qkv_col(t, HD) : t, c2 = permuted ? qkv_col(t + half, HD) : t + half; // where the pair sits in the GEMM's output
    int Ntot = (nH + 2 * nKV) * HD, pos = rowPos[m];
    // everything this thread will need from memory is requested up front: one latency instead of a chain of them
    const int slotRow = rowSlot[m];
    const double invf = invFreq[t];
    const float *src = P + (size_t)(m >> 5) * pStride + (size_t)(m & 31) * Ntot + (size_t)head * HD; // M-tile m/32, row m%32
    float x1 = src[c1], x2 = src[c2];
    float b1 = 0.f, b2 = 0.f;
    if (bias) b1 = bias[head * HD + t], b2 = bias[head * HD + t + half];
    for (int s0 = 1; s0 < splits; s0 += 8) { // ascending split order; eight splits' loads in flight together
        float a1[8], a2[8];
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (s0 + j < splits) a1[j] = src[(size_t)(s0 + j) * 32 * Ntot + c1], a2[j] = src[(size_t)(s0 + j) * 32 * Ntot + c2];
#pragma unroll
        for (int j = 0; j < 8; j++)
            if (s0 + j < splits) x1 = __fadd_rn(x1, a1[j]), x2 = __fadd_rn(x2, a2[j]);
    }
    if (bias) x1 = __fadd_rn(x1, b1), x2 = __fadd_rn(x2, b2);
    const int blkPre = tables[(size_t)slotRow * tabStride + (pos >> 6)];
    bool isQ = head < nH, isK = !isQ && head < nH + nKV;
    const float *nw = isQ ? qnorm : (isK ? knorm : nullptr);
    if (nw) { // RMSNorm over the head's HD values, f64 sum of squares
        double ss = (double)x1 * x1 + (double)x2 * x2;
        for (int o = half >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
        float inv = (float)(1.0 / sqrt(ss / (double)HD + (double)eps));
        x1 = __fmul_rn(__fmul_rn(x1, inv), nw[t]);
        x2 = __fmul_rn(__fmul_rn(x2, inv), nw[t + half]);
    }
    float o1 = x1, o2 = x2;
    if (isQ || isK) {
        double theta = __dmul_rn((double)pos, invf);
        double c = cos(theta), s = sin(theta);
        o1 = rope_first(x1, x2, c, s);
        o2 = rope_second(x1, x2, c, s);
    }
    if (isQ) {
        float *dst = q + (size_t)m * nH * HD + (size_t)head * HD;
        dst[t] = o1;
        dst[t + half] = o2;
        return;
    }
    int kvh = isK ? head - nH : head - nH - nKV;
    int blk = blkPre, p = pos & 63;
    size_t region = ((size_t)blk * nKV + kvh) * 64 * HD;
    if constexpr (I8) {
        // one scale per (position, kv head): the head's largest magnitude over all its rotation pairs (block = one head)
        float ma = fmaxf(fabsf(o1), fabsf(o2));
        for (int o = half >> 1; o > 0; o >>= 1) ma = fmaxf(ma, __shfl_xor(ma, o, 64));
        float inv, sc = kv8_scale(ma, &inv);
        unsigned char *dst8 = (unsigned char *)(isK ? KpV : VpV) + region;
        dst8[isK ? k8_index(HD, p, t) : v8_index(HD, p, t)] = kv8_code(o1, inv);
        dst8[isK ? k8_index(HD, p, t + half) : v8_index(HD, p, t + half)] = kv8_code(o2, inv);
        if (t == 0) (isK ? Ksc : Vsc)[((size_t)blk * nKV + kvh) * 64 + p] = sc;
        return;
    }
    uint16_t *dstp = (uint16_t *)(isK ? KpV : VpV);
    for (int e = 0; e < 2; e++) {
        int d = e ? t + half : t;
        int idx = isK ? (HD == 128 ? k_elem_index<128>(p, d) : k_elem_index<64>(p, d)) : (HD == 128 ? v_elem_index<128>(p, d) : v_elem_index<64>(p, d));
        dstp[region + idx] = f32_to_f16_half_up(e ? o2 : o1);
    }
}

extern "C" __global__ void rd_k_qkv_rope_store(const float *__restrict__ P, int splits, float *__restrict__ q, uint16_t *__restrict__ Kp,
                                               uint16_t *__restrict__ Vp, const int *__restrict__ tables, int tabStride,
                                               const int *__restrict__ rowSlot, const int *__restrict__ rowPos, const double *__restrict__ invFreq,
                                               const float *__restrict__ qnorm, const float *__restrict__ knorm, float eps, int nH, int nKV, int HD,
                                               size_t pStride, const float *__restrict__ bias, int permuted) {
    qkv_rope_store_body<false>(P, splits, q, Kp, Vp, nullptr, nullptr, tables, tabStride, rowSlot, rowPos, invFreq, qnorm, knorm, eps, nH, nKV, HD, pStride, bias, permuted);
}
// The same into the int8 cache: the K or V head is quantized with its own scale after RoPE (backend/cuda/kv8_store.cu).
extern "C" __global__ void rd_k_qkv_rope_store_i8(const float *__restrict__ P, int splits, float *__restrict__ q, signed char *__restrict__ Kp,
                                                  signed char *__restrict__ Vp, float *__restrict__ Ksc, float *__restrict__ Vsc,
                                                  const int *__restrict__ tables, int tabStride, const int *__restrict__ rowSlot,
                                                  const int *__restrict__ rowPos, const double *__restrict__ invFreq, const float *__restrict__ qnorm,
                                                  const float *__restrict__ knorm, float eps, int nH, int nKV, int HD, size_t pStride, const float *__restrict__ bias,
                                                  int permuted) {
    qkv_rope_store_body<true>(P, splits, q, Kp, Vp, Ksc, Vsc, tables, tabStride, rowSlot, rowPos, invFreq, qnorm, knorm, eps, nH, nKV, HD, pStride, bias, permuted);
}

typedef float float4v __attribute__((ext_vector_type(4)));

// tanh(x) = 1 - 2 / (e^(2x) + 1), with the hardware exponential and reciprocal: absolute error below 1e-6 over the whole
// range (the argument is clamped where the result is 1 to the last bit anyway), far inside the attention bar.
__device__ __forceinline__ float fast_tanh(float x) {
    x = fminf(12.f, fmaxf(-12.f, x));
    float t = __expf(2.f * x);
    return 1.f - 2.f * __frcp_rn(t + 1.f);
}

__device__ __forceinline__ float ld_part(const float *p) { return *p; }

// rd_k_attn_partial_wide runs this many waves a block, each wave on its own item; the other attention kernels one
#define RD_ATTN_BLOCK_WAVES 4
struct AttnItem {
    int row, kvh, b0, b1; // first row, kv head (low 16 bits) and number of rows (high 16 bits), block range [b0,b1) of the sequence
};

// One wave per item: online-softmax attention of the G query heads of one kv head over blocks [b0,b1) of one sequence.
// Scores: S = Q.K^T on 16x16x32 f16 MFMA with Q split into hi+lo halves (K is exactly f16), so dots carry f32 accuracy.
// P.V likewise with P split hi+lo. Writes unnormalised (O, m, l) per head: part[item][G][HD+2].
// I8: K and V are int8 codes with one f32 scale per (key, kv head). A code is exactly an f16, so the same MFMAs run on the
// codes; the key's K scale multiplies its finished scores and its V scale multiplies its probabilities before the P.V product:
// sum_d q_d (c_d s) = s sum_d q_d c_d and sum_key p (c s) = sum_key (p s) c, which is the dequantized arithmetic up to f32 rounding.
// ROWS: an item covers up to 16/G consecutive positions of one sequence (rows row..row+n-1 of the step, lengths len..len+n-1, all
// with the same number of blocks): the 16 rows of the A operand hold (position j, head g) at j*G + g, every K and V fragment
// is read once for all of them, and each row masks the keys past its own length. A row's arithmetic is what it would be in
// an item of its own: a unit in which all of its keys are masked leaves its maximum, sum and output untouched (factor 1, p = 0).
// Partials: part[item][16][HD+2] instead of part[item][G][HD+2].
// eight stored bytes (code + 128) -> eight f16 codes, exactly: under a 0x64 high byte a byte u is 1024 + u; minus 1152.
__device__ __forceinline__ half8_t kv8_to_half8(uint32_t w0, uint32_t w1) {
    const half2_t off = {(half_t)(-1152.f), (half_t)(-1152.f)};
    uint32_t u0 = __builtin_amdgcn_perm(0x64646464u, w0, 0x04010400u), u1 = __builtin_amdgcn_perm(0x64646464u, w0, 0x04030402u);
    uint32_t u2 = __builtin_amdgcn_perm(0x64646464u, w1, 0x04010400u), u3 = __builtin_amdgcn_perm(0x64646464u, w1, 0x04030402u);
    half2_t v0, v1, v2, v3;
    __builtin_memcpy(&v0, &u0, 4);
    __builtin_memcpy(&v1, &u1, 4);
    __builtin_memcpy(&v2, &u2, 4);
    __builtin_memcpy(&v3, &u3, 4);
    v0 += off, v1 += off, v2 += off, v3 += off;
    return (half8_t){v0.x, v0.y, v1.x, v1.y, v2.x, v2.y, v3.x, v3.y};
}

// A wave's lanes exchange the probabilities through their own 2 KB of LDS: one wave's LDS operations complete in the order they
// were issued, so ordering them for the compiler (and draining the wave's own LDS counter) is all the hand-off needs. A block-wide
// barrier would be wrong here: the waves of a block work on different items with different trip counts.
#define RD_WAVE_LDS_SYNC()                                       \
    do {                                                         \
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");   \
        __builtin_amdgcn_wave_barrier();                         \
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");   \
    } while (0)

// The work on one unit of 32 keys whose K and V fragments (KF, VF) and int8 scales (KS, VS) are in registers: scores, online softmax
// with a lazy rescale of the running output (only when some row's maximum moved: a factor of exactly 1 changes nothing; a key
// past a row's end has no scale to trust, so its probability is zeroed rather than scaled), P.V. A macro, not a function, so
// that the unit loops below expand to the same statements wherever they use it. Uses the enclosing kernel body's names.
#define RD_ATTN_UNIT(KF, VF, KS, VS, KEY0) \
    { \
        float4v S[2];                                                                                                                                  \
        _Pragma("unroll")                                                                                                                              \
        for (int t = 0; t < 2; t++) {                                                                                                                  \
            S[t] = (float4v){0.f, 0.f, 0.f, 0.f};                                                                                                      \
        _Pragma("unroll")                                                                                                                              \
            for (int c = 0; c < NC; c++) {                                                                                                             \
                half8_t kb;                                                                                                                            \
                if constexpr (I8)                                                                                                                      \
                    kb = kv8_to_half8(KF[t][c >> 1][(c & 1) * 2], KF[t][c >> 1][(c & 1) * 2 + 1]);                                                     \
                else                                                                                                                                   \
                    __builtin_memcpy(&kb, &KF[t][c], 16);                                                                                              \
                S[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(qhi[c], kb, S[t], 0, 0, 0);                                                              \
                S[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(qlo[c], kb, S[t], 0, 0, 0);                                                              \
            }                                                                                                                                          \
        }                                                                                                                                              \
        float mx[4];                                                                                                                                   \
        _Pragma("unroll")                                                                                                                              \
        for (int r = 0; r < 4; r++) {                                                                                                                  \
            mx[r] = -INFINITY;                                                                                                                         \
        _Pragma("unroll")                                                                                                                              \
            for (int t = 0; t < 2; t++) {                                                                                                              \
                float s = S[t][r] * scale;                                                                                                             \
                if constexpr (I8) s = S[t][r] * KS[t] * scale;                                                                                         \
                if (softcap != 0.f) s = softcap * fast_tanh(s * rcap);                                                                                 \
                if ((KEY0) + t * 16 + l16 >= lenr[r] || (KEY0) + t * 16 + l16 < startr[r]) s = -INFINITY;                                           \
                S[t][r] = s;                                                                                                                           \
                mx[r] = fmaxf(mx[r], s);                                                                                                               \
            }                                                                                                                                          \
            mx[r] = group_max16(mx[r]);                                                                                                                \
        }                                                                                                                                              \
        float alpha[4];                                                                                                                                \
        _Pragma("unroll")                                                                                                                              \
        for (int r = 0; r < 4; r++) {                                                                                                                  \
            float mn = fmaxf(mrun[r], mx[r]);                                                                                                          \
            const bool none = mn == -INFINITY; /* no key of this row yet (all before its window): nothing moves */                                     \
            alpha[r] = none ? 1.f : __expf(mrun[r] - mn);                                                                                              \
            mrun[r] = mn;                                                                                                                              \
            float ps = 0.f;                                                                                                                            \
        _Pragma("unroll")                                                                                                                              \
            for (int t = 0; t < 2; t++) {                                                                                                              \
                float p = none ? 0.f : __expf(S[t][r] - mn);                                                                                           \
                ps += p;                                                                                                                               \
                if constexpr (I8) p = ((KEY0) + t * 16 + l16 < lenr[r] && (KEY0) + t * 16 + l16 >= startr[r]) ? p * VS[t] : 0.f;                       \
                half_t hi = (half_t)p;                                                                                                                 \
                int idx = (4 * lg + r) * 32 + t * 16 + l16;                                                                                            \
                pbuf[idx] = hi;                                                                                                                        \
                pbuf[512 + idx] = (half_t)(p - (float)hi);                                                                                             \
            }                                                                                                                                          \
            lrun[r] = lrun[r] * alpha[r] + ps;                                                                                                         \
        }                                                                                                                                              \
        if (__builtin_amdgcn_ballot_w64(alpha[0] != 1.f || alpha[1] != 1.f || alpha[2] != 1.f || alpha[3] != 1.f) != 0) {                              \
        _Pragma("unroll")                                                                                                                              \
            for (int ct = 0; ct < NCT; ct++)                                                                                                           \
        _Pragma("unroll")                                                                                                                              \
                for (int r = 0; r < 4; r++) O[ct][r] *= alpha[r];                                                                                      \
        }                                                                                                                                              \
        RD_WAVE_LDS_SYNC();                                                                                                                                 \
        half8_t phi, plo;                                                                                                                              \
        {                                                                                                                                              \
            uint4_t a = *(const uint4_t *)(pbuf + l16 * 32 + lg * 8), bq = *(const uint4_t *)(pbuf + 512 + l16 * 32 + lg * 8);                         \
            __builtin_memcpy(&phi, &a, 16);                                                                                                            \
            __builtin_memcpy(&plo, &bq, 16);                                                                                                           \
        }                                                                                                                                              \
        RD_WAVE_LDS_SYNC();                                                                                                                                 \
        _Pragma("unroll")                                                                                                                              \
        for (int ct = 0; ct < NCT; ct++) {                                                                                                             \
            half8_t vb;                                                                                                                                \
            if constexpr (I8)                                                                                                                          \
                vb = kv8_to_half8(VF[ct >> 1][(ct & 1) * 2], VF[ct >> 1][(ct & 1) * 2 + 1]);                                                           \
            else                                                                                                                                       \
                __builtin_memcpy(&vb, &VF[ct], 16);                                                                                                    \
            O[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(phi, vb, O[ct], 0, 0, 0);                                                                   \
            O[ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(plo, vb, O[ct], 0, 0, 0);                                                                   \
        }                                                                                                                                              \
    }

template <int HD, bool I8, bool ROWS = false, bool DEEP = false, int DEEP_UNITS = 2>
__device__ __forceinline__ void attn_partial_body(const AttnItem *__restrict__ items, const int *__restrict__ rowLen, const int *__restrict__ rowSlot,
                                                  const int *__restrict__ tables, int tabStride, const void *__restrict__ KpV,
                                                  const void *__restrict__ VpV, const float *__restrict__ Ksc, const float *__restrict__ Vsc,
                                                  const float *__restrict__ q, float *__restrict__ part, int nH, int nKV, float scale,
                                                  float softcap, int window, half_t *pbuf) {
    constexpr int NC = HD / 32, NCT = HD / 16;
    constexpr int KL = I8 ? NC / 2 : NC, VL = I8 ? NCT / 2 : NCT; // 16-byte loads per key tile of K, per 32 keys of V
    constexpr int ELEM = I8 ? 1 : 2;
    // a block is one wave, or several waves on consecutive items of the list (a step's padded list: fewer, fatter blocks to dispatch)
    const int item = blockIdx.x * (int)(blockDim.x >> 6) + (int)(threadIdx.x >> 6);
    pbuf += (threadIdx.x >> 6) * 1024;
    AttnItem it = items[item];
    if (it.row < 0) return; // padding of the work list: names no row
    const int nrows = ROWS ? it.kvh >> 16 : 1;
    it.kvh &= 0xffff;
    const int lane = threadIdx.x & 63, l16 = lane & 15, lg = lane >> 4;
    const int G = nH / nKV, len0 = rowLen[it.row];
    const int len = len0 + nrows - 1; // the longest row's: the unit loop runs to it
    const int *tab = tables + (size_t)rowSlot[it.row] * tabStride;
    // head row a of the tile = (position a / G, head a % G); this lane loads Q for row l16 and owns score rows 4*lg + r
    const int qj = ROWS ? l16 / G : 0, qg = ROWS ? l16 - qj * G : l16;
    // window > 0 (a sliding-window layer; kvmgr.WindowNeedStart): a row at position p = len-1 reads keys p-window+1 .. p only
    int lenr[4], startr[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        lenr[r] = ROWS ? len0 + min((4 * lg + r) / G, nrows - 1) : len;
        startr[r] = window > 0 ? max(lenr[r] - window, 0) : 0;
    }

    // Q fragments (A operand): lane (head row l16, d quarter lg)
    half8_t qhi[NC], qlo[NC];
#pragma unroll
    for (int c = 0; c < NC; c++) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float v = 0.f;
            if (ROWS ? qj < nrows : l16 < G) v = q[(size_t)(it.row + qj) * nH * HD + (size_t)(it.kvh * G + qg) * HD + lg * (HD / 4) + c * 8 + i];
            half_t hi = (half_t)v;
            qhi[c][i] = hi;
            qlo[c][i] = (half_t)(v - (float)hi);
        }
    }
    float4v O[NCT];
#pragma unroll
    for (int ct = 0; ct < NCT; ct++) O[ct] = (float4v){0.f, 0.f, 0.f, 0.f};
    float mrun[4], lrun[4];
#pragma unroll
    for (int r = 0; r < 4; r++) mrun[r] = -INFINITY, lrun[r] = 0.f;
    const float rcap = softcap != 0.f ? 1.f / softcap : 0.f;

    const size_t regionBytes = (size_t)64 * HD * ELEM;
    if constexpr (DEEP) {
        // DEEP_UNITS units in flight per wave: unit i+DEEP_UNITS is requested as soon as unit i has been worked on, so a wave that has the SIMD
        // to itself overlaps its memory latency with its own arithmetic. For steps whose work list leaves most SIMDs one wave
        // (few or short sequences); the units are worked on in the same order, so the results are the plain loop's bit for bit.
        struct Unit {
            uint4_t kf[2][KL], vf[VL];
            float ks[2], vs[2];
        };
        const int nU = min(2 * (it.b1 - it.b0), (len - it.b0 * 64 + 31) >> 5); // units with a key of the longest row
        auto load_unit = [&](Unit &un, int i) {
            const int blk = tab[it.b0 + (i >> 1)], u = i & 1;
            const uint4_t *Kr = (const uint4_t *)((const char *)KpV + ((size_t)blk * nKV + it.kvh) * regionBytes);
            const uint4_t *Vr = (const uint4_t *)((const char *)VpV + ((size_t)blk * nKV + it.kvh) * regionBytes);
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int c = 0; c < KL; c++) un.kf[t][c] = __builtin_nontemporal_load(Kr + ((u * 2 + t) * KL + c) * 64 + lane);
#pragma unroll
            for (int ct = 0; ct < VL; ct++) un.vf[ct] = __builtin_nontemporal_load(Vr + (u * VL + ct) * 64 + lane);
            un.ks[0] = un.ks[1] = un.vs[0] = un.vs[1] = 1.f;
            if constexpr (I8) {
                const size_t srow = ((size_t)blk * nKV + it.kvh) * 64;
#pragma unroll
                for (int t = 0; t < 2; t++) un.ks[t] = Ksc[srow + u * 32 + t * 16 + l16], un.vs[t] = Vsc[srow + u * 32 + t * 16 + l16];
            }
        };
        Unit un[DEEP_UNITS];
#pragma unroll
        for (int j = 0; j < DEEP_UNITS; j++)
            if (j < nU) load_unit(un[j], j);
        for (int i0 = 0; i0 < nU; i0 += DEEP_UNITS) {
#pragma unroll
            for (int j = 0; j < DEEP_UNITS; j++) {
                const int i = i0 + j;
                if (i < nU) {
                    const int key0 = (it.b0 + (i >> 1)) * 64 + (i & 1) * 32;
                    RD_ATTN_UNIT(un[j].kf, un[j].vf, un[j].ks, un[j].vs, key0)
                    if (i + DEEP_UNITS < nU) load_unit(un[j], i + DEEP_UNITS);
                }
            }
        }
    } else
    for (int b = it.b0; b < it.b1; b++) {
        const int blk = tab[b];
        const uint4_t *Kr = (const uint4_t *)((const char *)KpV + ((size_t)blk * nKV + it.kvh) * regionBytes);
        const uint4_t *Vr = (const uint4_t *)((const char *)VpV + ((size_t)blk * nKV + it.kvh) * regionBytes);
        const size_t srow = ((size_t)blk * nKV + it.kvh) * 64;
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int key0 = b * 64 + u * 32;
            if (key0 >= len) break;
            uint4_t kf[2][KL], vf[VL];
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int c = 0; c < KL; c++) kf[t][c] = __builtin_nontemporal_load(Kr + ((u * 2 + t) * KL + c) * 64 + lane);
#pragma unroll
            for (int ct = 0; ct < VL; ct++) vf[ct] = __builtin_nontemporal_load(Vr + (u * VL + ct) * 64 + lane);
            float ks[2] = {1.f, 1.f}, vs[2] = {1.f, 1.f}; // this lane's keys t*16 + l16
            if constexpr (I8) {
#pragma unroll
                for (int t = 0; t < 2; t++) ks[t] = Ksc[srow + u * 32 + t * 16 + l16], vs[t] = Vsc[srow + u * 32 + t * 16 + l16];
            }
            RD_ATTN_UNIT(kf, vf, ks, vs, key0)
        }
    }
    // lane (d column l16 of tile ct, head rows 4*lg+r): O[ct][r]; l partial sums live per key lane -> reduce over the 16 lanes
#pragma unroll
    for (int r = 0; r < 4; r++) {
        for (int o = 8; o > 0; o >>= 1) lrun[r] += __shfl_xor(lrun[r], o, 64);
        int g = 4 * lg + r;
        if (ROWS ? g < nrows * G : g < G) {
            float *dst = part + ((size_t)item * (ROWS ? 16 : G) + g) * (HD + 2);
#pragma unroll
            for (int ct = 0; ct < NCT; ct++) dst[ct * 16 + l16] = O[ct][r];
            if (l16 == 0) dst[HD] = mrun[r], dst[HD + 1] = lrun[r];
        }
    }
}

extern "C" __global__ __launch_bounds__(64) void rd_k_attn_partial(const AttnItem *__restrict__ items, const int *__restrict__ rowLen,
                                                                   const int *__restrict__ rowSlot, const int *__restrict__ tables, int tabStride,
                                                                   const uint16_t *__restrict__ Kp, const uint16_t *__restrict__ Vp,
                                                                   const float *__restrict__ q, float *__restrict__ part, int nH, int nKV, int HD,
                                                                   float scale, float softcap, int window) {
    __shared__ half_t pbuf[1024];
    if (HD == 128)
        attn_partial_body<128, false>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, nullptr, nullptr, q, part, nH, nKV, scale, softcap, window, pbuf);
    else
        attn_partial_body<64, false>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, nullptr, nullptr, q, part, nH, nKV, scale, softcap, window, pbuf);
}

// The same with four waves a block, each on its own item (grid = items / 4; the list is padded to whole blocks): for work lists of
// several waves per SIMD, where 4 096 one-wave blocks take the dispatcher longer than 1 024 fatter ones (61.0 against 62.2 us on one
// machine at 32 sequences of 512 to 4 096 keys; no difference at 16 384 items). A short list wants its waves spread over the
// compute units instead and keeps one wave a block.
extern "C" __global__ __launch_bounds__(64 * RD_ATTN_BLOCK_WAVES) void rd_k_attn_partial_wide(const AttnItem *__restrict__ items, const int *__restrict__ rowLen,
                                                                   const int *__restrict__ rowSlot, const int *__restrict__ tables, int tabStride,
                                                                   const uint16_t *__restrict__ Kp, const uint16_t *__restrict__ Vp,
                                                                   const float *__restrict__ q, float *__restrict__ part, int nH, int nKV, int HD,
                                                                   float scale, float softcap, int window) {
    __shared__ half_t pbuf[RD_ATTN_BLOCK_WAVES * 1024];
    if (HD == 128)
        attn_partial_body<128, false>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, nullptr, nullptr, q, part, nH, nKV, scale, softcap, window, pbuf);
    else
        attn_partial_body<64, false>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, nullptr, nullptr, q, part, nH, nKV, scale, softcap, window, pbuf);
}

// The same over the int8 cache: half the key/value bytes per launch.
extern "C" __global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(3, 3))) void rd_k_attn_partial_i8(const AttnItem *__restrict__ items, const int *__restrict__ rowLen,
                                                                      const int *__restrict__ rowSlot, const int *__restrict__ tables, int tabStride,
                                                                      const signed char *__restrict__ Kp, const signed char *__restrict__ Vp,
                                                                      const float *__restrict__ Ksc, const float *__restrict__ Vsc,
                                                                      const float *__restrict__ q, float *__restrict__ part, int nH, int nKV, int HD,
                                                                      float scale, float softcap, int window) {
    __shared__ half_t pbuf[1024];
    if (HD == 128)
        attn_partial_body<128, true>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, Ksc, Vsc, q, part, nH, nKV, scale, softcap, window, pbuf);
    else
        attn_partial_body<64, true>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, Ksc, Vsc, q, part, nH, nKV, scale, softcap, window, pbuf);
}

// The same two kernels with two units in flight per wave (see DEEP above), one wave per SIMD.
extern "C" __global__ __launch_bounds__(64) void rd_k_attn_partial_deep(const AttnItem *__restrict__ items, const int *__restrict__ rowLen,
                                                                        const int *__restrict__ rowSlot, const int *__restrict__ tables, int tabStride,
                                                                        const uint16_t *__restrict__ Kp, const uint16_t *__restrict__ Vp,
                                                                        const float *__restrict__ q, float *__restrict__ part, int nH, int nKV, int HD,
                                                                        float scale, float softcap, int window) {
    __shared__ half_t pbuf[1024];
    if (HD == 128)
        attn_partial_body<128, false, false, true>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, nullptr, nullptr, q, part, nH, nKV, scale, softcap, window, pbuf);
    else
        attn_partial_body<64, false, false, true>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, nullptr, nullptr, q, part, nH, nKV, scale, softcap, window, pbuf);
}

extern "C" __global__ __launch_bounds__(64) void rd_k_attn_partial_deep_i8(const AttnItem *__restrict__ items, const int *__restrict__ rowLen,
                                                                      const int *__restrict__ rowSlot, const int *__restrict__ tables, int tabStride,
                                                                      const signed char *__restrict__ Kp, const signed char *__restrict__ Vp,
                                                                      const float *__restrict__ Ksc, const float *__restrict__ Vsc,
                                                                      const float *__restrict__ q, float *__restrict__ part, int nH, int nKV, int HD,
                                                                      float scale, float softcap, int window) {
    __shared__ half_t pbuf[1024];
    if (HD == 128)
        attn_partial_body<128, true, false, true>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, Ksc, Vsc, q, part, nH, nKV, scale, softcap, window, pbuf);
    else
        attn_partial_body<64, true, false, true>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, Ksc, Vsc, q, part, nH, nKV, scale, softcap, window, pbuf);
}

// Items of several positions each (see ROWS above): steps that carry more than one row of a sequence — prompt passes, verification.
extern "C" __global__ __launch_bounds__(64) void rd_k_attn_partial_rows(const AttnItem *__restrict__ items, const int *__restrict__ rowLen,
                                                                        const int *__restrict__ rowSlot, const int *__restrict__ tables, int tabStride,
                                                                        const uint16_t *__restrict__ Kp, const uint16_t *__restrict__ Vp,
                                                                        const float *__restrict__ q, float *__restrict__ part, int nH, int nKV, int HD,
                                                                        float scale, float softcap, int window) {
    __shared__ half_t pbuf[1024];
    if (HD == 128)
        attn_partial_body<128, false, true>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, nullptr, nullptr, q, part, nH, nKV, scale, softcap, window, pbuf);
    else
        attn_partial_body<64, false, true>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, nullptr, nullptr, q, part, nH, nKV, scale, softcap, window, pbuf);
}

extern "C" __global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(3, 3))) void rd_k_attn_partial_rows_i8(const AttnItem *__restrict__ items, const int *__restrict__ rowLen,
                                                                      const int *__restrict__ rowSlot, const int *__restrict__ tables, int tabStride,
                                                                      const signed char *__restrict__ Kp, const signed char *__restrict__ Vp,
                                                                      const float *__restrict__ Ksc, const float *__restrict__ Vsc,
                                                                      const float *__restrict__ q, float *__restrict__ part, int nH, int nKV, int HD,
                                                                      float scale, float softcap, int window) {
    __shared__ half_t pbuf[1024];
    if (HD == 128)
        attn_partial_body<128, true, true>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, Ksc, Vsc, q, part, nH, nKV, scale, softcap, window, pbuf);
    else
        attn_partial_body<64, true, true>(items, rowLen, rowSlot, tables, tabStride, Kp, Vp, Ksc, Vsc, q, part, nH, nKV, scale, softcap, window, pbuf);
}

// Merge the partials of one (row, query head) in ascending item order (deterministic):
// out = sum O_i e^(m_i-M) / sum l_i e^(m_i-M). itemStart[3*(row*nKV+kvh)] and the entry after it bound that pair's items, the
// third entry is the row's place among the positions its items cover (0 where an item is one position); partRows is the
// number of head rows an item writes (G, or 16 from the kernels whose items cover several positions). Block = RD_ATTN_PIECES * HD/4 threads: thread (item i, quarter
// dq) brings four values of item i into LDS, so every item's load is in flight at once; the first HD/4 threads then fold
// the items in order. lds: RD_ATTN_PIECES*(HD+2) floats. Returns true in the threads that hold a result (four consecutive d).
#define RD_ATTN_PIECES 16
// sinks (may be NULL): one learned logit per query head that joins the softmax's maximum and denominator and nothing else
// (decoder/attention.go:305-322 sinkMax / sinkSum).
__device__ __forceinline__ bool attn_combine_block(const float *__restrict__ part, const int *__restrict__ itemStart, int partRows, int nH, int nKV,
                                                   int HD, int m, int head, float *lds, float *out, const float *__restrict__ sinks = nullptr) {
    const int Q = HD >> 2, ti = threadIdx.x / Q, dq = threadIdx.x - ti * Q;
    const int G = nH / nKV, kvh = head / G, g = head % G;
    const int *rg = itemStart + (m * nKV + kvh) * 3;
    const int i0 = rg[0], n = rg[1] - i0, sub = rg[2];
    const size_t stride = (size_t)partRows * (HD + 2);
    const float *p0 = part + ((size_t)i0 * partRows + sub * G + g) * (HD + 2);
    float *vals = lds, *mm = lds + RD_ATTN_PIECES * HD, *ll = mm + RD_ATTN_PIECES;
    // A sequence of up to 128 blocks has at most RD_ATTN_PIECES items: one round. A longer one has more (its items stay short so
    // that even a lone long sequence spreads over the chip): the maximum over all of them first, then rounds of RD_ATTN_PIECES
    // folded in the same ascending order with the same arithmetic.
    float M = -INFINITY;
    if (n > RD_ATTN_PIECES) {
        for (int i = threadIdx.x; i < n; i += blockDim.x) M = fmaxf(M, p0[(size_t)i * stride + HD]);
        for (int o = 32; o > 0; o >>= 1) M = fmaxf(M, __shfl_xor(M, o, 64));
        if ((threadIdx.x & 63) == 0) mm[threadIdx.x >> 6] = M; // at most 8 waves: fits the 16 floats of mm
        __syncthreads();
        M = -INFINITY;
        for (int w = 0; w < (int)(blockDim.x >> 6); w++) M = fmaxf(M, mm[w]);
        if (sinks) M = fmaxf(M, sinks[head]);
        __syncthreads(); // mm is reused by the rounds
    }
    float num[4] = {0.f, 0.f, 0.f, 0.f}, den = 0.f;
    for (int base = 0; base < n; base += RD_ATTN_PIECES) {
        const int nb = min(n - base, RD_ATTN_PIECES);
        if (ti < nb) {
            const float *p = p0 + (size_t)(base + ti) * stride;
            const float2 a = *(const float2 *)(p + dq * 4), b = *(const float2 *)(p + dq * 4 + 2); // rows are 8-byte aligned (HD+2 is even)
            float *v = vals + ti * HD + dq * 4;
            v[0] = a.x, v[1] = a.y, v[2] = b.x, v[3] = b.y;
            if (dq == 0) mm[ti] = p[HD], ll[ti] = p[HD + 1];
        }
        __syncthreads();
        if (ti == 0) {
            if (n <= RD_ATTN_PIECES) {
                for (int i = 0; i < nb; i++) M = fmaxf(M, mm[i]);
                if (sinks) M = fmaxf(M, sinks[head]);
            }
            for (int i = 0; i < nb; i++) {
                const float *v = vals + i * HD + dq * 4;
                const float w = __expf(mm[i] - M);
                num[0] = fmaf(v[0], w, num[0]), num[1] = fmaf(v[1], w, num[1]), num[2] = fmaf(v[2], w, num[2]), num[3] = fmaf(v[3], w, num[3]);
                den = fmaf(ll[i], w, den);
            }
        }
        if (base + RD_ATTN_PIECES < n) __syncthreads(); // the next round overwrites what the folding threads read
    }
    if (ti != 0) return false;
    if (sinks) den += __expf(sinks[head] - M);
#pragma unroll
    for (int e = 0; e < 4; e++) out[e] = num[e] / den;
    return true;
}

// Grid (nH, rows), block RD_ATTN_PIECES * HD/4.
extern "C" __global__ __launch_bounds__(512) void rd_k_attn_combine(const float *__restrict__ part, const int *__restrict__ itemStart, int partRows,
                                                                     float *__restrict__ out, int nH, int nKV, int HD, const float *__restrict__ sinks) {
    __shared__ float lds[RD_ATTN_PIECES * (128 + 2)];
    const int head = blockIdx.x, m = blockIdx.y;
    float v[4];
    if (attn_combine_block(part, itemStart, partRows, nH, nKV, HD, m, head, lds, v, sinks)) {
        float *o = out + (size_t)m * nH * HD + (size_t)head * HD + threadIdx.x * 4;
        o[0] = v[0], o[1] = v[1], o[2] = v[2], o[3] = v[3];
    }
}
