// gemm8.h — the decode GEMMs in the reference's own arithmetic: int8 activation codes x integer weight codes on the int8
// matrix cores, an exact int32 dot per group of 32, folded in f32 by the group's two scales
// (goinfer backend/cuda/actgroup.cu:298-355 rowQ4K: facc += idot_g * ((d*sc_g) * aS_g); facc += -(dmin*m_g) * asum_g).
//
// Activations arrive as A8 blocks (a8.h): int8 codes in MFMA operand order, a scale and a scaled code sum per group of 32.
//
// One MFMA gives the 32x32 int32 dots of one group (32 batch rows x 32 weight rows). The products of the two scales, one per
// (batch row, weight row, group), are an outer product: v_mfma_f32_32x32x1_2b_f32 forms them for two groups at once in the
// accumulator layout, so the fold costs a convert and an fma per output and group. The -dmin*m term is a small f32 matrix
// product over the groups and rides v_mfma_f32_32x32x2_f32 into the same accumulators.
//
// A block is KW waves per 32-row weight tile, each on its own K range with its own operands straight from global memory (no
// LDS staging, no barrier in the loop); their partial sums are folded through LDS in ascending wave order. The order of every
// output's sum is fixed by (split, wave, super-block, group) and independent of M: a row in a batch is the row alone, bit for bit.
#pragma once
#include "act.h"
#include "attn.h"

typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x32_t __attribute__((ext_vector_type(32)));

// A8 blocks back to rows, for checking what a producer wrote: codes int8 [M][K], scales and sums f32 [M][K/32].
// Grid (ceil(K/256), M), block 256.
extern "C" __global__ void rd_k_unpack_act8(const uint8_t *__restrict__ A8, signed char *__restrict__ codes, float *__restrict__ scales,
                                            float *__restrict__ sums, int K) {
    const int m = blockIdx.y, k = blockIdx.x * 256 + threadIdx.x;
    if (k >= K) return;
    codes[(size_t)m * K + k] = (signed char)A8[a8_code_offset(m, k)];
    if ((k & 31) == 0) {
        const uint8_t *p = A8 + a8_scale_offset(m, k >> 5);
        scales[(size_t)m * (K >> 5) + (k >> 5)] = *(const float *)p;
        sums[(size_t)m * (K >> 5) + (k >> 5)] = *(const float *)(p + (RD_A8_SUMS - RD_A8_SCALES));
    }
}

// A8 blocks as the values a consumer multiplies: out[m][k] = code * scale (f32). Grid (ceil(K/256), M), block 256.
extern "C" __global__ void rd_k_unpanel_a8(const uint8_t *__restrict__ A8, float *__restrict__ out, int K) {
    const int m = blockIdx.y, k = blockIdx.x * 256 + threadIdx.x;
    if (k >= K) return;
    out[(size_t)m * K + k] = __fmul_rn((float)(signed char)A8[a8_code_offset(m, k)], *(const float *)(A8 + a8_scale_offset(m, k >> 5)));
}

// Operands are read through buffer descriptors that cover exactly the K range of the wave: a prefetch past the end of the range
// is answered with zeros by the address check and touches no memory, so the loop issues every load unconditionally and the
// compiler's count of loads in flight stays exact (a branch around a load makes it wait for everything).
typedef __amdgpu_buffer_rsrc_t rd_rsrc_t;
__device__ __forceinline__ rd_rsrc_t make_rsrc(const void *p, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(p), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint4_t buf_load16(rd_rsrc_t r, int voff, int imm) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, voff + imm, 0, 0);
}
__device__ __forceinline__ uint4_t buf_load16_nt(rd_rsrc_t r, int voff, int imm) { // streamed once: weights
    return __builtin_amdgcn_raw_buffer_load_b128(r, voff + imm, 0, 2);
}

struct A8Regs {
    uint4_t c[8];
    float4_t as, asum;
};
// voff: byte offset of the block inside the descriptor's range plus lane * 16
__device__ __forceinline__ void a8_load(A8Regs &a, rd_rsrc_t r, int voff) {
#pragma unroll
    for (int g = 0; g < 8; g++) a.c[g] = buf_load16(r, voff, g * 1024);
    uint4_t s = buf_load16(r, voff, RD_A8_SCALES), u = buf_load16(r, voff, RD_A8_SUMS);
    __builtin_memcpy(&a.as, &s, 16);
    __builtin_memcpy(&a.asum, &u, 16);
}

__device__ __forceinline__ i32x4_t as_i32x4(uint4_t v) {
    i32x4_t r;
    __builtin_memcpy(&r, &v, 16);
    return r;
}

// acc += fold of one group's dots: a convert and an fma per output (the scale products come from the matrix core). NR: how many
// of the tile's sixteen accumulator registers hold batch rows in use: register r of lane half h is batch row (r>>2)*8 + h*4 + (r&3),
// so a batch of at most 8 rows lives in registers 0..3 and the fold of the other twelve, three quarters of the kernel's
// VALU work, is left out (their sums are never stored).
#define RD_FOLD(ACC, DOT, S, OFF, NR)                                                  \
    _Pragma("unroll") for (int r_ = 0; r_ < (NR); r_++) ACC[r_] = __builtin_fmaf((float)DOT[r_], S[(OFF) + r_], ACC[r_]);

// The two lane halves' values of x on every lane: lo = lanes 0..31's, hi = lanes 32..63's (v_permlane32_swap).
__device__ __forceinline__ void halves_i(int x, int &lo, int &hi) {
    const auto r = __builtin_amdgcn_permlane32_swap((unsigned)x, (unsigned)x, false, false);
    lo = (int)r[0], hi = (int)r[1];
}
__device__ __forceinline__ void halves_f(float x, float &lo, float &hi) {
    int a, b;
    halves_i(__float_as_int(x), a, b);
    lo = __int_as_float(a), hi = __int_as_float(b);
}
__device__ __forceinline__ int halves_sum(int x) {
    int a, b;
    halves_i(x, a, b);
    return a + b;
}

// ---------------- Q4_K ----------------
// Tile of 32 rows x one super-block, 4608 B: the 32 headers (16 B: d, dmin, 12 scale bytes), then four planes [64 lanes][16 B]:
// plane p, lane (row r, half h) holds raw code bytes [32p + 16h, +16) of row r, i.e. elements 16h..16h+15 of sub-block 2p in
// the low nibbles and of sub-block 2p+1 in the high nibbles. Same bytes as the file, same 4.5 bits per weight.
extern "C" __global__ void rd_k_retile_q4k8(const uint8_t *__restrict__ raw, uint8_t *__restrict__ tiled, int N, int nSB) {
    const int tile = blockIdx.x, sb = blockIdx.y, t = threadIdx.x; // 288 x 16 B
    if (t >= 288) return;
    uint8_t *dst = tiled + ((size_t)tile * nSB + sb) * 4608;
    const uint4_t *src;
    if (t < 32) {
        src = (const uint4_t *)(raw + ((size_t)(tile * 32 + t) * nSB + sb) * 144);
    } else {
        const int u = t - 32, p = u >> 6, lane = u & 63, r = lane & 31, h = lane >> 5;
        src = (const uint4_t *)(raw + ((size_t)(tile * 32 + r) * nSB + sb) * 144 + 16 + p * 32 + h * 16);
    }
    *(uint4_t *)(dst + (size_t)t * 16) = *src;
}

struct Q4K8Tile {
    uint4_t hdr, q[4];
};

struct Q4K8Traits {
    typedef Q4K8Tile Tile;
    static constexpr int TILE_BYTES = 4608;
    // off: byte offset of the tile inside the descriptor's range
    static __device__ __forceinline__ void load(Tile &w, rd_rsrc_t r, int off, int lane) {
        w.hdr = buf_load16_nt(r, off + (lane & 31) * 16, 0);
#pragma unroll
        for (int c = 0; c < 4; c++) w.q[c] = buf_load16_nt(r, off + lane * 16, 512 + c * 1024);
    }
    // Lane (n, h) decodes the scales of sub-blocks 2p+h, p = 0..3: dsc = d * sc, ndm = -(dmin * m). The 6-bit fields are cut out
    // with the lane half folded into the bit offset (one v_bfe_u32 a field), not as both halves' values and a select.
    static __device__ __forceinline__ void decode(const Tile &w, int h, float (&dsc)[4], float (&ndm)[4]) {
        const uint32_t y = w.hdr.y, z = w.hdr.z, x = w.hdr.w, hx = w.hdr.x;
        half2_t dd;
        __builtin_memcpy(&dd, &hx, 4);
        const float d = (float)dd.x, dmin = (float)dd.y;
        const uint32_t h8 = (uint32_t)h << 3;
#pragma unroll
        for (int p = 0; p < 4; p++) {
            uint32_t sc, mn;
            if (p < 2) { // sub-blocks 0..3: the low six bits of bytes 0..3 of the scale and the minimum word
                const uint32_t j8 = 16u * p + h8;
                sc = __builtin_amdgcn_ubfe(y, j8, 6u), mn = __builtin_amdgcn_ubfe(z, j8, 6u);
            } else { // sub-blocks 4..7: a nibble of the third word and the top two bits of the matching byte
                const uint32_t j8 = 16u * (p - 2) + h8;
                sc = __builtin_amdgcn_ubfe(x, j8, 4u) | (__builtin_amdgcn_ubfe(y, j8 + 6u, 2u) << 4);
                mn = __builtin_amdgcn_ubfe(x, j8 + 4u, 4u) | (__builtin_amdgcn_ubfe(z, j8 + 6u, 2u) << 4);
            }
            dsc[p] = __fmul_rn(d, (float)sc);
            ndm[p] = -__fmul_rn(dmin, (float)mn);
        }
    }
    // acc[m][n] += sum over the super-block's 8 groups: the lane half is the block index of the two-block scale product and the k
    // index of the minimum product.
    template <int NR> static __device__ __forceinline__ void mma(float16_t &acc, const Tile &w, const A8Regs &a, const void *, int, int lane) {
        float dsc[4], ndm[4];
        decode(w, lane >> 5, dsc, ndm);
        const f32x32_t zero32 = {0.f};
        const i32x16_t zero16 = {0};
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const f32x32_t s2 = __builtin_amdgcn_mfma_f32_32x32x1f32(a.as[p], dsc[p], zero32, 0, 0, 0);
            const uint4_t raw = w.q[p];
            uint4_t lo, hi;
#pragma unroll
            for (int i = 0; i < 4; i++) lo[i] = raw[i] & 0x0F0F0F0Fu, hi[i] = (raw[i] >> 4) & 0x0F0F0F0Fu;
            const i32x16_t d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[2 * p]), as_i32x4(lo), zero16, 0, 0, 0);
            const i32x16_t d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[2 * p + 1]), as_i32x4(hi), zero16, 0, 0, 0);
            RD_FOLD(acc, d0, s2, 0, NR)
            RD_FOLD(acc, d1, s2, 16, NR)
        }
#pragma unroll
        for (int p = 0; p < 4; p++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.asum[p], ndm[p], acc, 0, 0, 0);
    }
    // The same sums for ONE batch row on the vector ALU (a step of one sequence: goinfer's Forward). `a` holds row 0's operands
    // broadcast: lane (n, h) has the row's codes 16h..16h+15 of every group and the scale and sum of groups 2p+h, beside its
    // own weight row's codes and sub-block scales for the same elements and groups. A group's dot is the two lane halves'
    // sixteen-element dots added (v_dot4_i32_i8, exact); the fold is the matrix-core path's own chain, operation for operation:
    // its scale product is one rounded multiply (v_mfma_f32_32x32x1 with a zero accumulator gives exactly that), its groups are
    // folded in ascending order with one fma each, and v_mfma_f32_32x32x2 is fma(a1, b1, fma(a0, b0, c)), k ascending — measured
    // on 204 800 random outputs, no exception. The row is therefore the row a batch gives, bit for bit; the tests that compare a
    // batched row with its solo run hold the two paths to that. Both lane halves compute the chain (accumulator 0 of the upper half
    // is batch row 4, which a one-row step never stores).
    static constexpr bool GEMV1 = true;
    static __device__ __forceinline__ void mma1(float16_t &acc, const Tile &w, const A8Regs &a, const void *, int, int lane) {
        float dsc[4], ndm[4];
        decode(w, lane >> 5, dsc, ndm);
        fold1(acc, w, a, dsc, ndm);
    }
    // dsc[p], ndm[p]: this lane's scale and negated minimum of group 2p + (lane half); codes 0..15 in the tile's nibbles
    static __device__ __forceinline__ void fold1(float16_t &acc, const Tile &w, const A8Regs &a, const float (&dsc)[4], const float (&ndm)[4]) {
        float f = acc[0];
        float se[4], so[4];
#pragma unroll
        for (int p = 0; p < 4; p++) halves_f(__fmul_rn(a.as[p], dsc[p]), se[p], so[p]);
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint4_t raw = w.q[p];
            int x0 = 0, x1 = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                x0 = __builtin_amdgcn_sdot4((int)(raw[i] & 0x0F0F0F0Fu), (int)a.c[2 * p][i], x0, false);
                x1 = __builtin_amdgcn_sdot4((int)((raw[i] >> 4) & 0x0F0F0F0Fu), (int)a.c[2 * p + 1][i], x1, false);
            }
            f = __builtin_fmaf((float)halves_sum(x0), se[p], f);
            f = __builtin_fmaf((float)halves_sum(x1), so[p], f);
        }
#pragma unroll
        for (int p = 0; p < 4; p++) {
            float ae, ao, ne, no;
            halves_f(a.asum[p], ae, ao);
            halves_f(ndm[p], ne, no);
            f = __builtin_fmaf(ae, ne, f);
            f = __builtin_fmaf(ao, no, f);
        }
        acc[0] = f;
    }
    static constexpr bool INT_ACC = false;
    static __device__ __forceinline__ void finish(float16_t &, const void *, const uint8_t *, int, int) {}
};

// ---------------- W8A8: int8 codes, one f32 scale per row (goinfer WeightMat.Int8; backend/cuda/actgroup.cu:283-288,421-437) ----------------
// Tile of 32 rows x 256 k, 8192 B: eight planes [64 lanes][16 B], plane g lane (row r, half h) = codes of elements 16h..16h+15 of
// group g of the block. K is padded to a multiple of 256 with zero codes. facc += idot_g * aS_g; dst = facc * wScale[n].
extern "C" __global__ __launch_bounds__(512) void rd_k_retile_w8a8_8(const uint8_t *__restrict__ raw, uint8_t *__restrict__ tiled, int N, int K) {
    const int tile = blockIdx.x, kb = blockIdx.y, t = threadIdx.x; // 512 x 16 B
    const int g = t >> 6, lane = t & 63, r = lane & 31, h = lane >> 5, k0 = kb * 256 + g * 32 + h * 16;
    uint4_t v = {0u, 0u, 0u, 0u};
    if (k0 < K) v = *(const uint4_t *)(raw + (size_t)(tile * 32 + r) * K + k0); // K % 32 == 0: a 16-byte run is inside K or past it
    *(uint4_t *)(tiled + ((size_t)tile * gridDim.y + kb) * 8192 + (size_t)t * 16) = v;
}

struct W8Tile8 {
    uint4_t q[8];
};
struct W8A8Traits8 {
    typedef W8Tile8 Tile;
    // One batch row on the vector ALU (see Q4K8Traits::mma1): the scale "product with one" is the scale itself, the chain the same.
    static constexpr bool GEMV1 = true;
    static __device__ __forceinline__ void mma1(float16_t &acc, const Tile &w, const A8Regs &a, const void *, int, int) {
        float f = acc[0];
#pragma unroll
        for (int p = 0; p < 4; p++) {
            float se, so;
            halves_f(a.as[p], se, so);
            int x0 = 0, x1 = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                x0 = __builtin_amdgcn_sdot4((int)w.q[2 * p][i], (int)a.c[2 * p][i], x0, false);
                x1 = __builtin_amdgcn_sdot4((int)w.q[2 * p + 1][i], (int)a.c[2 * p + 1][i], x1, false);
            }
            f = __builtin_fmaf((float)halves_sum(x0), se, f);
            f = __builtin_fmaf((float)halves_sum(x1), so, f);
        }
        acc[0] = f;
    }
    static constexpr int TILE_BYTES = 8192;
    static __device__ __forceinline__ void load(Tile &w, rd_rsrc_t r, int off, int lane) {
#pragma unroll
        for (int g = 0; g < 8; g++) w.q[g] = buf_load16_nt(r, off + lane * 16 + (g >> 2) * 4096, (g & 3) * 1024);
    }
    template <int NR> static __device__ __forceinline__ void mma(float16_t &acc, const Tile &w, const A8Regs &a, const void *, int, int lane) {
        const f32x32_t zero32 = {0.f};
        const i32x16_t zero16 = {0};
#pragma unroll
        for (int p = 0; p < 4; p++) {
            // the activation scale of every (batch row, group) spread over the accumulator layout: a product with one
            const f32x32_t s2 = __builtin_amdgcn_mfma_f32_32x32x1f32(a.as[p], 1.f, zero32, 0, 0, 0);
            const i32x16_t d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[2 * p]), as_i32x4(w.q[2 * p]), zero16, 0, 0, 0);
            const i32x16_t d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[2 * p + 1]), as_i32x4(w.q[2 * p + 1]), zero16, 0, 0, 0);
            RD_FOLD(acc, d0, s2, 0, NR)
            RD_FOLD(acc, d1, s2, 16, NR)
        }
    }
    static constexpr bool INT_ACC = false;
    static __device__ __forceinline__ void finish(float16_t &acc, const void *aux, const uint8_t *, int tile, int lane) {
        const float ws = ((const float *)aux)[tile * 32 + (lane & 31)];
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = mul_rounded(acc[r], ws);
    }
};

// The scale of batch row m of an M-tile whose activations carry one scale per row (ActQuantGroup 0): the row's scale sits in
// every group slot of its A8 blocks; the first block's first slot is read.
__device__ __forceinline__ float a8_row_scale(const uint8_t *__restrict__ A8, int m) { return *(const float *)(A8 + a8_scale_offset(m, 0)); }

// W8A8 with one activation scale per row (goinfer's ActQuantGroup 0, the lane its staged QuantBackend.MatmulW8A8 hook serves:
// decoder/backend.go:38-46, weightmat.go:931-947; device twin internal/gpudev/gemv_quant.cu:99-112): the int32 dot runs over the
// whole of K, exactly, on the matrix core's own accumulator (no fold in the loop at all), and the result is
// dst = (f32(idot) * aS[m]) * wScale[n], two rounded multiplies: linalg.MatmulBTW8A8 bit for bit, whatever the order of the
// partial dots. The sixteen accumulators are int32 values kept in the float registers' bits.
struct W8A8RowTraits8 {
    typedef W8Tile8 Tile;
    static constexpr int TILE_BYTES = 8192;
    static constexpr bool GEMV1 = true, INT_ACC = true;
    static __device__ __forceinline__ void load(Tile &w, rd_rsrc_t r, int off, int lane) { W8A8Traits8::load(w, r, off, lane); }
    template <int NR> static __device__ __forceinline__ void mma(float16_t &acc, const Tile &w, const A8Regs &a, const void *, int, int) {
        i32x16_t d = __builtin_bit_cast(i32x16_t, acc);
#pragma unroll
        for (int g = 0; g < 8; g++) d = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[g]), as_i32x4(w.q[g]), d, 0, 0, 0);
        acc = __builtin_bit_cast(float16_t, d);
    }
    static __device__ __forceinline__ void mma1(float16_t &acc, const Tile &w, const A8Regs &a, const void *, int, int) {
        int x = 0;
#pragma unroll
        for (int g = 0; g < 8; g++)
#pragma unroll
            for (int i = 0; i < 4; i++) x = __builtin_amdgcn_sdot4((int)w.q[g][i], (int)a.c[g][i], x, false);
        acc[0] = __int_as_float(__float_as_int(acc[0]) + halves_sum(x));
    }
    static __device__ __forceinline__ void finish(float16_t &acc, const void *aux, const uint8_t *A8, int tile, int lane) {
        const float ws = ((const float *)aux)[tile * 32 + (lane & 31)];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            acc[r] = mul_rounded(mul_rounded((float)__float_as_int(acc[r]), a8_row_scale(A8, m)), ws);
        }
    }
};

// ---------------- W4A8: canonical int4 nibbles (value nib-8), binary16 scale per 32 (decoder/weightmat.go:160-178) ----------------
// Tile of 32 rows x 256 k, 4608 B, the Q4_K tile's shape: 32 headers of 16 B (the row's eight group scales, f16), then four planes
// [64 lanes][16 B]: plane p, lane (row r, half h), byte b = element 16h+b of group 2p in the low nibble and of group 2p+1 in the
// high nibble (re-packed from the canonical order, element k in nibble k%2 of byte k/2, at upload). The dot runs on the stored
// nibbles (0..15) and the -8 comes back as a term in the activation sums, exactly as Q4_K's minimum does:
// sum_k (nib-8)*a = sum_k nib*a - 8*sum_k a, so  facc += ws_g*aS_g*idot_g;  facc += -(8*ws_g)*asum_g.  K padded to 256 with zeros.
extern "C" __global__ __launch_bounds__(320) void rd_k_retile_w4a8_8(const uint8_t *__restrict__ nib, const uint16_t *__restrict__ s16,
                                                                      uint8_t *__restrict__ tiled, int N, int K) {
    const int tile = blockIdx.x, kb = blockIdx.y, t = threadIdx.x; // 288 x 16 B
    if (t >= 288) return;
    uint8_t *dst = tiled + ((size_t)tile * gridDim.y + kb) * 4608;
    const int nG = K >> 5;
    uint4_t v = {0u, 0u, 0u, 0u};
    if (t < 32) {
        uint16_t sc[8];
#pragma unroll
        for (int j = 0; j < 8; j++) sc[j] = kb * 8 + j < nG ? s16[(size_t)(tile * 32 + t) * nG + kb * 8 + j] : (uint16_t)0;
        __builtin_memcpy(&v, sc, 16);
    } else {
        const int u = t - 32, p = u >> 6, lane = u & 63, r = lane & 31, h = lane >> 5;
        const uint8_t *row = nib + (size_t)(tile * 32 + r) * (K >> 1);
        uint8_t by[16];
#pragma unroll
        for (int b = 0; b < 16; b++) {
            const int klo = kb * 256 + (2 * p) * 32 + h * 16 + b, khi = klo + 32;
            const int lo = klo < K ? (row[klo >> 1] >> (4 * (klo & 1))) & 15 : 8, hi = khi < K ? (row[khi >> 1] >> (4 * (khi & 1))) & 15 : 8;
            by[b] = (uint8_t)(lo | (hi << 4));
        }
        __builtin_memcpy(&v, by, 16);
    }
    *(uint4_t *)(dst + (size_t)t * 16) = v;
}

struct W4A8Traits8 {
    typedef Q4K8Tile Tile;
    static constexpr int TILE_BYTES = 4608;
    static constexpr bool GEMV1 = true;
    static __device__ __forceinline__ void mma1(float16_t &acc, const Tile &w, const A8Regs &a, const void *, int, int lane) {
        const int h = lane >> 5;
        float dsc[4], ndm[4];
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint32_t wd = w.hdr[p];
            dsc[p] = f16_bits_to_f32((uint16_t)(h ? wd >> 16 : wd & 0xffffu));
            ndm[p] = -8.f * dsc[p];
        }
        Q4K8Traits::fold1(acc, w, a, dsc, ndm);
    }
    static __device__ __forceinline__ void load(Tile &w, rd_rsrc_t r, int off, int lane) { Q4K8Traits::load(w, r, off, lane); }
    template <int NR> static __device__ __forceinline__ void mma(float16_t &acc, const Tile &w, const A8Regs &a, const void *, int, int lane) {
        const int h = lane >> 5;
        float dsc[4], ndm[4];
#pragma unroll
        for (int p = 0; p < 4; p++) { // the scale of group 2p+h: half h of header word p
            const uint32_t wd = w.hdr[p];
            dsc[p] = f16_bits_to_f32((uint16_t)(h ? wd >> 16 : wd & 0xffffu));
            ndm[p] = -8.f * dsc[p];
        }
        const f32x32_t zero32 = {0.f};
        const i32x16_t zero16 = {0};
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const f32x32_t s2 = __builtin_amdgcn_mfma_f32_32x32x1f32(a.as[p], dsc[p], zero32, 0, 0, 0);
            const uint4_t raw = w.q[p];
            uint4_t lo, hi;
#pragma unroll
            for (int i = 0; i < 4; i++) lo[i] = raw[i] & 0x0F0F0F0Fu, hi[i] = (raw[i] >> 4) & 0x0F0F0F0Fu;
            const i32x16_t d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[2 * p]), as_i32x4(lo), zero16, 0, 0, 0);
            const i32x16_t d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[2 * p + 1]), as_i32x4(hi), zero16, 0, 0, 0);
            RD_FOLD(acc, d0, s2, 0, NR)
            RD_FOLD(acc, d1, s2, 16, NR)
        }
#pragma unroll
        for (int p = 0; p < 4; p++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.asum[p], ndm[p], acc, 0, 0, 0);
    }
    static constexpr bool INT_ACC = false;
    static __device__ __forceinline__ void finish(float16_t &, const void *, const uint8_t *, int, int) {}
};

// W4A8 with one activation scale per row (ActQuantGroup 0, the lane goinfer's staged QuantBackend4.MatmulW4A8 hook and its expert
// kernels serve: decoder/backend.go:55-75, weightmat.go:904-912; device twins internal/gpudev/gemv_quant.cu:40-95,
// backend/cuda/moe_rows.cu:24-106): per group of 32 facc = fma(f32(idot_g), ws_g, facc) with the signed dot of nib-8, and
// dst = facc * aS[m] at the end. The stored nibble xor 8 is the two's-complement nibble of nib-8; at the top of a byte it is the
// int8 16*(nib-8), so the matrix core's dot is 16 times the group's, exactly, and the 1/16 rides in the scale (a power of two:
// the fma sees the same real product). The weight scale belongs to the lane (its column), so there is no scale outer product
// and no sum term: eight int8 MFMAs a block and a convert and an fma per output and group.
struct W4A8RowTraits8 {
    typedef Q4K8Tile Tile;
    static constexpr int TILE_BYTES = 4608;
    static constexpr bool GEMV1 = true, INT_ACC = false;
    static __device__ __forceinline__ void load(Tile &w, rd_rsrc_t r, int off, int lane) { Q4K8Traits::load(w, r, off, lane); }
    static __device__ __forceinline__ void scales(const Tile &w, int p, float &s0, float &s1) { // groups 2p and 2p+1 of the lane's column, / 16
        const uint32_t wd = w.hdr[p];
        s0 = f16_bits_to_f32((uint16_t)(wd & 0xffffu)) * 0.0625f, s1 = f16_bits_to_f32((uint16_t)(wd >> 16)) * 0.0625f;
    }
    template <int NR> static __device__ __forceinline__ void mma(float16_t &acc, const Tile &w, const A8Regs &a, const void *, int, int) {
        const i32x16_t zero16 = {0};
#pragma unroll
        for (int p = 0; p < 4; p++) {
            uint4_t lo, hi;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t x = w.q[p][i] ^ 0x88888888u;
                lo[i] = (x << 4) & 0xF0F0F0F0u, hi[i] = x & 0xF0F0F0F0u;
            }
            float s0, s1;
            scales(w, p, s0, s1);
            const i32x16_t d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[2 * p]), as_i32x4(lo), zero16, 0, 0, 0);
            const i32x16_t d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[2 * p + 1]), as_i32x4(hi), zero16, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < NR; r++) acc[r] = __builtin_fmaf((float)d0[r], s0, acc[r]);
#pragma unroll
            for (int r = 0; r < NR; r++) acc[r] = __builtin_fmaf((float)d1[r], s1, acc[r]);
        }
    }
    // one batch row on the vector ALU: the same chain (group 2p, then 2p+1, one fma each), the dot from the two lane halves
    static __device__ __forceinline__ void mma1(float16_t &acc, const Tile &w, const A8Regs &a, const void *, int, int) {
        float f = acc[0];
#pragma unroll
        for (int p = 0; p < 4; p++) {
            int x0 = 0, x1 = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t x = w.q[p][i] ^ 0x88888888u;
                x0 = __builtin_amdgcn_sdot4((int)((x << 4) & 0xF0F0F0F0u), (int)a.c[2 * p][i], x0, false);
                x1 = __builtin_amdgcn_sdot4((int)(x & 0xF0F0F0F0u), (int)a.c[2 * p + 1][i], x1, false);
            }
            float s0, s1;
            scales(w, p, s0, s1);
            f = __builtin_fmaf((float)halves_sum(x0), s0, f);
            f = __builtin_fmaf((float)halves_sum(x1), s1, f);
        }
        acc[0] = f;
    }
    static __device__ __forceinline__ void finish(float16_t &acc, const void *, const uint8_t *A8, int, int lane) {
#pragma unroll
        for (int r = 0; r < 16; r++) acc[r] = mul_rounded(acc[r], a8_row_scale(A8, (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3)));
    }
};

// The K loop of one wave: two weight tiles and two activation blocks in registers, each refilled with the block two ahead as soon as
// it has been multiplied. Loads are counted in issue order by the wave's wait counter, so a block's activations are asked for
// before its weights: waiting for activations then never waits for younger weight tiles. The refills are unconditional (past
// the end of the range the descriptor answers with zeros and touches no memory): only the second product of a round sits under
// a branch, so the compiler's count of the loads in flight stays exact.
// NR: accumulator registers folded (RD_FOLD). aoff: the lane's byte offset inside an activation block, lane * 16 for batch row
// lane & 31 (a caller that gathers rows passes the offset of another row, or one past every block for a row with no source:
// the descriptor then answers zeros).
// NR == 1: one batch row on the vector ALU (traits with GEMV1), else NR accumulator registers folded from the matrix core's dots
template <class T, int NR>
__device__ __forceinline__ void gemm8_mma(float16_t &acc, const typename T::Tile &w, const A8Regs &a, const void *aux, int tile, int lane) {
    if constexpr (NR == 1)
        T::mma1(acc, w, a, aux, tile, lane);
    else
        T::template mma<NR>(acc, w, a, aux, tile, lane);
}

template <class T, int NR = 16>
__device__ __forceinline__ void gemm8_wave_loop(float16_t &acc, const uint8_t *__restrict__ wb, const uint8_t *__restrict__ ab, int nk, const void *aux,
                                                int tile, int lane, int aoff) {
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
    if (nk <= 0) return;
    constexpr int AB = RD_A8_BLOCK_BYTES;
    const rd_rsrc_t wr = make_rsrc(wb, (uint32_t)nk * T::TILE_BYTES), ar = make_rsrc(ab, (uint32_t)nk * AB);
    if constexpr (NR == 1) aoff = (lane >> 5) * 512; // batch row 0's operands on every lane of a half (see mma1)
    typename T::Tile w0, w1;
    A8Regs a0, a1;
    a8_load(a0, ar, aoff);
    T::load(w0, wr, 0, lane);
    a8_load(a1, ar, AB + aoff);
    T::load(w1, wr, T::TILE_BYTES, lane);
    for (int it = 0; it < nk; it += 2) {
        gemm8_mma<T, NR>(acc, w0, a0, aux, tile, lane);
        a8_load(a0, ar, (it + 2) * AB + aoff);
        T::load(w0, wr, (it + 2) * T::TILE_BYTES, lane);
        if (it + 1 < nk) gemm8_mma<T, NR>(acc, w1, a1, aux, tile, lane);
        a8_load(a1, ar, (it + 3) * AB + aoff);
        T::load(w1, wr, (it + 3) * T::TILE_BYTES, lane);
    }
}

// A one-row step whose norm-and-quantize kernel is folded into the projection (norm_row0_to_lds): the row's operands come from the
// block's LDS image instead of the A8 panel. The registers get what a8_load gives a one-row wave (batch row 0's sixteen codes of
// every group on each lane half, the scales and sums of the half's four groups), so mma1 forms the same sums from them.
struct Row0Norm {
    const float *hIn; // the residual row
    float *hOut;      // the row after the pending add (another buffer: other blocks still read hIn)
    const float *P;   // the pending split-K partials [splits][32][H] (row 0 of each), or null
    const float *w;   // norm weights
    int splits, H;
    float eps;
};
__device__ __forceinline__ void a8_row0_from_lds(A8Regs &a, const uint8_t *img, int kb, int h) {
    const uint8_t *p = img + (size_t)kb * RD_ROW0_KB_BYTES;
#pragma unroll
    for (int g = 0; g < 8; g++) a.c[g] = *(const uint4_t *)(p + g * 32 + h * 16);
    a.as = *(const float4_t *)(p + 256 + h * 16);
    a.asum = *(const float4_t *)(p + 288 + h * 16);
}
// DEPTH weight tiles are in flight per wave (two: four were measured slower on the gate|up shape, 21.2 against 20.1 us a launch).
// w[]: the range's first DEPTH tiles, asked for by the caller before the row was formed. kb0: the range's first K-block.
template <class T, int DEPTH>
__device__ __forceinline__ void gemm8_wave_loop_row0(float16_t &acc, typename T::Tile (&w)[DEPTH], rd_rsrc_t wr, const uint8_t *img, int kb0, int nk,
                                                     const void *aux, int tile, int lane) {
    const int h = lane >> 5;
    for (int it = 0; it < nk; it += DEPTH) {
#pragma unroll
        for (int i = 0; i < DEPTH; i++) {
            if (it + i < nk) {
                A8Regs a;
                a8_row0_from_lds(a, img, kb0 + it + i, h);
                T::mma1(acc, w[i], a, aux, tile, lane);
            }
            T::load(w[i], wr, (it + i + DEPTH) * T::TILE_BYTES, lane); // past the range: answered with zeros, never used
        }
    }
}
// The projection's K loop for a one-row step with the norm folded in: weights first, then the row, then the loop.
template <class T, int BS, int DEPTH>
__device__ __forceinline__ void gemm8_row0_norm_loop(float16_t &acc, const uint8_t *__restrict__ wb, int kb0, int nk, const Row0Norm &rn, bool writesRow,
                                                     uint8_t *img, double *red, const void *aux, int tile, int lane) {
#pragma unroll
    for (int i = 0; i < 16; i++) acc[i] = 0.f;
    const rd_rsrc_t wr = make_rsrc(wb, (uint32_t)nk * T::TILE_BYTES);
    typename T::Tile w[DEPTH];
#pragma unroll
    for (int i = 0; i < DEPTH; i++) T::load(w[i], wr, i * T::TILE_BYTES, lane);
    norm_row0_to_lds<BS>(rn.hIn, writesRow ? rn.hOut : nullptr, rn.P, rn.splits, rn.w, rn.eps, rn.H, img, red);
    gemm8_wave_loop_row0<T, DEPTH>(acc, w, wr, img, kb0, nk, aux, tile, lane);
}

// Folds the KW waves' partial sums of each tile into the tile's first wave, ascending wave order, through LDS
// (xch: TPB*(KW-1)*1024 floats). Every wave of the block calls it.
template <int KW, int TPB, bool INT_ACC = false>
__device__ __forceinline__ void gemm8_fold_waves(float16_t &acc, float *xch) {
    if constexpr (KW > 1) {
        const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, t = wave / KW, kw = wave % KW;
        float4_t *x4 = (float4_t *)xch;
        if (kw > 0) {
#pragma unroll
            for (int q = 0; q < 4; q++) x4[((t * (KW - 1) + kw - 1) * 4 + q) * 64 + lane] = (float4_t){acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]};
        }
        __syncthreads();
        if (kw == 0) {
#pragma unroll
            for (int k2 = 1; k2 < KW; k2++)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float4_t v = x4[((t * (KW - 1) + k2 - 1) * 4 + q) * 64 + lane];
                    if constexpr (INT_ACC) { // int32 partial dots in the registers' bits: exact in any order
#pragma unroll
                        for (int e = 0; e < 4; e++) acc[4 * q + e] = __int_as_float(__float_as_int(acc[4 * q + e]) + __float_as_int(v[e]));
                    } else {
                        acc[4 * q] += v.x, acc[4 * q + 1] += v.y, acc[4 * q + 2] += v.z, acc[4 * q + 3] += v.w;
                    }
                }
        }
    }
}

// Grid (ceil(N/(32*TPB)), splits), block KW*TPB waves. P[split][32][ldP] receives the sums of K-blocks [split*kbPerSplit, +kbPerSplit).
// resid != NULL (splits must be 1): the sums are added to resid[m][n] in place instead (the residual stream), nothing goes to P.
template <class T, int KW, int TPB, int NR = 16>
__device__ __forceinline__ void gemm8_body(const uint8_t *__restrict__ Wt, const void *__restrict__ aux, const uint8_t *__restrict__ A8,
                                           float *__restrict__ P, int N, int nKB, int kbPerSplit, int M, int ldP, float *__restrict__ resid, float *lds) {
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int tile = blockIdx.x * TPB + wave / KW, kw = wave % KW, split = blockIdx.y;
    const int kb0 = split * kbPerSplit, kb1 = min(nKB, kb0 + kbPerSplit);
    const int per = (max(kb1 - kb0, 0) + KW - 1) / KW;
    const int s0 = kb0 + kw * per, nk = max(0, min(kb1, s0 + per) - s0);
    const bool active = tile * 32 < N;
    float16_t acc;
    gemm8_wave_loop<T, NR>(acc, Wt + ((size_t)(active ? tile : 0) * nKB + s0) * T::TILE_BYTES, A8 + (size_t)s0 * RD_A8_BLOCK_BYTES,
                           active ? nk : 0, aux, tile, lane, lane * 16);
    gemm8_fold_waves<KW, TPB, T::INT_ACC>(acc, lds);
    if (!active || kw != 0) return;
    T::finish(acc, aux, A8, tile, lane);
    const int n = tile * 32 + (lane & 31);
    if (resid) {
        float old[16]; // all sixteen reads in flight before the first add
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            old[r] = resid[(size_t)min(m, M - 1) * ldP + n];
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            if (m < M) resid[(size_t)m * ldP + n] = __fadd_rn(old[r], acc[r]);
        }
        return;
    }
    float *out = P + (size_t)split * 32 * ldP + n;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (m < M) out[(size_t)m * ldP] = acc[r];
    }
}

// Rows past 32 are further M-tiles of 32, one per grid.z: M-tile z reads its activations a8Stride bytes further on and writes its
// sums pStride floats further on; the tiles of a launch are independent and a row's sums do not depend on how many there are.
#define RD_GEMM8_KERNEL(NAME, TRAITS, KW, TPB)                                                                                                       \
    extern "C" __global__ __launch_bounds__(64 * KW * TPB) void NAME(const uint8_t *__restrict__ Wt, const void *__restrict__ aux,                   \
                                                                     const uint8_t *__restrict__ A8, float *__restrict__ P, int N, int nKB,         \
                                                                     int kbPerSplit, int M, int ldP, float *__restrict__ resid, size_t a8Stride,   \
                                                                     size_t pStride) {                                                              \
        __shared__ float lds[(KW > 1 ? TPB * (KW - 1) * 1024 : 1)];                                                                                  \
        const int z = blockIdx.z;                                                                                                                    \
        A8 += (size_t)z * a8Stride, P += (size_t)z * pStride, M = min(32, M - 32 * z);                                                               \
        if (resid) resid += (size_t)z * 32 * ldP;                                                                                                    \
        /* up to 8 batch rows live in four accumulator registers, up to 16 in eight: the fold of the others is left out */                          \
        if (TRAITS::GEMV1 && M == 1) /* one row: the same sums on the vector ALU */                                                                  \
            gemm8_body<TRAITS, KW, TPB, 1>(Wt, aux, A8, P, N, nKB, kbPerSplit, M, ldP, resid, lds);                                                  \
        else if (M <= 8)                                                                                                                             \
            gemm8_body<TRAITS, KW, TPB, 4>(Wt, aux, A8, P, N, nKB, kbPerSplit, M, ldP, resid, lds);                                                  \
        else if (M <= 16)                                                                                                                            \
            gemm8_body<TRAITS, KW, TPB, 8>(Wt, aux, A8, P, N, nKB, kbPerSplit, M, ldP, resid, lds);                                                  \
        else                                                                                                                                         \
            gemm8_body<TRAITS, KW, TPB, 16>(Wt, aux, A8, P, N, nKB, kbPerSplit, M, ldP, resid, lds);                                                 \
    }

RD_GEMM8_KERNEL(rd_k_gemm8_q4k_kw2, Q4K8Traits, 2, 2)
RD_GEMM8_KERNEL(rd_k_gemm8_q4k_kw4, Q4K8Traits, 4, 1)
RD_GEMM8_KERNEL(rd_k_gemm8_q4k_kw8, Q4K8Traits, 8, 1)
RD_GEMM8_KERNEL(rd_k_gemm8_w8a8_kw2, W8A8Traits8, 2, 2)
RD_GEMM8_KERNEL(rd_k_gemm8_w8a8_kw4, W8A8Traits8, 4, 1)
RD_GEMM8_KERNEL(rd_k_gemm8_w8a8_kw8, W8A8Traits8, 8, 1)
RD_GEMM8_KERNEL(rd_k_gemm8_w4a8_kw2, W4A8Traits8, 2, 2)
RD_GEMM8_KERNEL(rd_k_gemm8_w4a8_kw4, W4A8Traits8, 4, 1)
RD_GEMM8_KERNEL(rd_k_gemm8_w4a8_kw8, W4A8Traits8, 8, 1)
// one activation scale per row (ActQuantGroup 0); launched with one split: the row scale is applied to the finished sum
RD_GEMM8_KERNEL(rd_k_gemm8_w8a8r_kw2, W8A8RowTraits8, 2, 2)
RD_GEMM8_KERNEL(rd_k_gemm8_w8a8r_kw4, W8A8RowTraits8, 4, 1)
RD_GEMM8_KERNEL(rd_k_gemm8_w8a8r_kw8, W8A8RowTraits8, 8, 1)
RD_GEMM8_KERNEL(rd_k_gemm8_w4a8r_kw2, W4A8RowTraits8, 2, 2)
RD_GEMM8_KERNEL(rd_k_gemm8_w4a8r_kw4, W4A8RowTraits8, 4, 1)
RD_GEMM8_KERNEL(rd_k_gemm8_w4a8r_kw8, W4A8RowTraits8, 8, 1)

// ---------------- fused gate|up projection + SwiGLU + per-32 quantization ----------------
// goinfer decoder/cpu_gateup_fused.go:83-148 in one launch. W holds [gate rows; up rows] (2*I rows). Grid (I/32), block 2*KW waves:
// waves 0..KW-1 own gate tile t over K (each its own range), waves KW..2KW-1 the matching up tile. After the fold both finished
// tiles meet in LDS in accumulator order, and every wave takes its share of the sixteen accumulator registers: in that order a
// half-wave holds the 32 columns of one batch row, which is exactly one activation group of the down projection, so
// silu(gate)*up (silu in f64, decoder/rmsnorm.go:204-207) is quantized where it sits and written in the layout the down projection reads.
// The K loop, its wave ranges and the fold are those of the plain kernel with the same KW: the sums are the same bits.
template <class T, int KW, int NR = 16, int ACT = 0, bool NORM = false>
__device__ __forceinline__ void gemm8_gateup_body(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ A8, uint8_t *__restrict__ XpOut, int outKind,
                                                  int I, int nKB, int M, float *lds, const Row0Norm *rn = nullptr, uint8_t *img = nullptr,
                                                  double *red = nullptr) {
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int half = wave / KW, kw = wave % KW, t = blockIdx.x, nGate = I >> 5, tile = half * nGate + t;
    const int per = (nKB + KW - 1) / KW, s0 = kw * per, nk = max(0, min(nKB, s0 + per) - s0);
    float16_t acc;
    if constexpr (NORM) // one row, its norm-and-quantize folded in (NR == 1)
        gemm8_row0_norm_loop<T, 128 * KW, 2>(acc, Wt + ((size_t)tile * nKB + s0) * T::TILE_BYTES, s0, nk, *rn, blockIdx.x == 0, img, red, nullptr, tile, lane);
    else
        gemm8_wave_loop<T, NR>(acc, Wt + ((size_t)tile * nKB + s0) * T::TILE_BYTES, A8 + (size_t)s0 * RD_A8_BLOCK_BYTES, nk, nullptr, tile, lane, lane * 16);
    gemm8_fold_waves<KW, 2>(acc, lds);
    __syncthreads(); // the fold area is read; it now takes the two finished tiles as [gate | up][register][lane]
    if (kw == 0) {
#pragma unroll
        for (int r = 0; r < 16; r++) lds[(half * 16 + r) * 64 + lane] = acc[r];
    }
    __syncthreads();
    constexpr int RPW = 16 / (2 * KW); // accumulator registers per wave
    const int n = t * 32 + (lane & 31);
#pragma unroll
    for (int j = 0; j < RPW; j++) {
        const int r = wave * RPW + j;
        const int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (r >= NR) continue; // batch rows past M: nothing folded, nothing to store
        const float a = __fmul_rn(gate_act(lds[r * 64 + lane], ACT), lds[(16 + r) * 64 + lane]);
        const Quant1 q = quant_one(a);
        if (outKind == RD_PANEL_A8) {
            // four neighbouring lanes hold four consecutive elements of the row: their codes leave as one word
            const int c = q.code & 255;
            const uint32_t word = (uint32_t)dpp_i<0x00>(c) | ((uint32_t)dpp_i<0x55>(c) << 8) | ((uint32_t)dpp_i<0xAA>(c) << 16) | ((uint32_t)dpp_i<0xFF>(c) << 24);
            if (m < M && (lane & 3) == 0) a8_store4(XpOut, m, n, word, q.sc, q.gsum);
        } else if (m < M) {
            panel_store(XpOut, outKind, m, n, q);
        }
    }
}

// grid.z: M-tiles of 32 rows, a8Stride / outStride bytes apart in the activations read and written. The _gelu kernel is the
// same with Gemma's geluTanh(gate)*up instead of silu(gate)*up.
#define RD_GEMM8_GATEUP_KERNEL(NAME, ACT)                                                                                                         \
    extern "C" __global__ __launch_bounds__(256) void NAME(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ A8, uint8_t *__restrict__ XpOut, \
                                                           int outKind, int I, int nKB, int M, size_t a8Stride, size_t outStride) {            \
        __shared__ float lds[2 * 1024];                                                                                                           \
        A8 += (size_t)blockIdx.z * a8Stride, XpOut += (size_t)blockIdx.z * outStride, M = min(32, M - 32 * (int)blockIdx.z);                      \
        if (M == 1)                                                                                                                               \
            gemm8_gateup_body<Q4K8Traits, 2, 1, ACT>(Wt, A8, XpOut, outKind, I, nKB, M, lds);                                                     \
        else if (M <= 8)                                                                                                                          \
            gemm8_gateup_body<Q4K8Traits, 2, 4, ACT>(Wt, A8, XpOut, outKind, I, nKB, M, lds);                                                     \
        else if (M <= 16)                                                                                                                         \
            gemm8_gateup_body<Q4K8Traits, 2, 8, ACT>(Wt, A8, XpOut, outKind, I, nKB, M, lds);                                                     \
        else                                                                                                                                      \
            gemm8_gateup_body<Q4K8Traits, 2, 16, ACT>(Wt, A8, XpOut, outKind, I, nKB, M, lds);                                                    \
    }
RD_GEMM8_GATEUP_KERNEL(rd_k_gemm8_q4k_gateup, 0)
RD_GEMM8_GATEUP_KERNEL(rd_k_gemm8_q4k_gateup_gelu, 1)
// A one-row step's gate|up projection with the norm-and-quantize kernel that feeds it folded in: every block forms the row
// (hIn + the pending partials, RMSNorm, per-32 quantization; norm_row0_to_lds) while its first weight tiles are on their way,
// block 0 writes the updated residual row to hOut, and the loop, the fold and the epilogue are the one-row kernel's own: the
// same bits as rd_k_add_rmsnorm_quant followed by rd_k_gemm8_q4k_gateup, in one launch less. Grid (I/32), block 256.
#define RD_GEMM8_GATEUP_NORM1_KERNEL(NAME, ACT)                                                                                                   \
    extern "C" __global__ __launch_bounds__(256) void NAME(const uint8_t *__restrict__ Wt, uint8_t *__restrict__ XpOut, int outKind, int I, int nKB, \
                                                           const float *__restrict__ hIn, float *__restrict__ hOut, const float *__restrict__ P,  \
                                                           int splits, const float *__restrict__ w, float eps, int H) {                          \
        __shared__ float lds[2 * 1024];                                                                                                           \
        __shared__ __align__(16) uint8_t img[16 * RD_ROW0_KB_BYTES];                                                                              \
        __shared__ double red[16];                                                                                                                \
        const Row0Norm rn{hIn, hOut, P, w, splits, H, eps};                                                                                       \
        gemm8_gateup_body<Q4K8Traits, 2, 1, ACT, true>(Wt, nullptr, XpOut, outKind, I, nKB, 1, lds, &rn, img, red);                               \
    }
RD_GEMM8_GATEUP_NORM1_KERNEL(rd_k_gemm8_q4k_gateup_norm1, 0)
RD_GEMM8_GATEUP_NORM1_KERNEL(rd_k_gemm8_q4k_gateup_gelu_norm1, 1)

// ---------------- q|k|v projection with bias, RoPE and the KV store in its epilogue ----------------
// The plain kernel with one split and, instead of the store of the sums, what rd_k_qkv_rope_store does to them (same arithmetic,
// same bits): the weight's rows are ordered so that a rotation pair sits in one tile, sixteen lanes apart (qkv_col), the angles'
// cos and sin come from the step's table, q goes to the f32 buffer and k, v to the row's position in the f16 pool. For models
// without QK-norm on the f16 cache. Grid (N/32, 1, M-tiles of 32 rows), block KW waves; M: the step's rows.
struct QkvEpilogue {
    float *q;
    uint16_t *Kp, *Vp;
    const int *tables, *rowSlot, *rowPos;
    const double2 *cs;
    const float *bias;
    int tabStride, nH, nKV, HD, row0;
};
template <class T, int KW, int NR = 16, bool NORM = false>
__device__ __forceinline__ void gemm8_qkv_body(const uint8_t *__restrict__ Wt, const void *__restrict__ aux, const uint8_t *__restrict__ A8, int N, int nKB,
                                               int M, const QkvEpilogue &e, float *lds, const Row0Norm *rn = nullptr, uint8_t *img = nullptr,
                                               double *red = nullptr) {
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int tile = blockIdx.x, kw = wave;
    const int per = (nKB + KW - 1) / KW, s0 = kw * per, nk = max(0, min(nKB, s0 + per) - s0);
    const int HD = e.HD, half = HD >> 1, head = (tile * 32) / HD, j = ((tile * 32) % HD) >> 5;
    const bool isQ = head < e.nH, isK = !isQ && head < e.nH + e.nKV;
    // The epilogue belongs to the whole block: the tile's 32 rows x 16 rotation pairs are dealt over its threads, PPT pairs each
    // (thread t takes pair t & 15 of rows t >> 4, + 4*KW, ...), so no wave runs more than a few dozen instructions of it.
    // What a thread needs from memory for its pairs is asked for ahead of time: the row's place in the cache (two dependent loads)
    // before the K loop, the angle and the bias after it, ahead of the fold.
    constexpr int PPT = 512 / (64 * KW);
    const int pi = tid & 15, d1 = 16 * j + pi, d2 = half + d1; // this thread's pair: elements d1, d2 of the head, columns pi, pi + 16 of the tile
    int where[PPT];                                            // block * 64 + position in the block
    if (!isQ) {
#pragma unroll
        for (int i = 0; i < PPT; i++) {
            const int m = e.row0 + min((tid >> 4) + 4 * KW * i, M - 1), pos = e.rowPos[m];
            where[i] = e.tables[(size_t)e.rowSlot[m] * e.tabStride + (pos >> 6)] * 64 + (pos & 63);
        }
    }
    float16_t acc;
    if constexpr (NORM) // one row, its norm-and-quantize folded in (NR == 1)
        gemm8_row0_norm_loop<T, 64 * KW, 2>(acc, Wt + ((size_t)tile * nKB + s0) * T::TILE_BYTES, s0, nk, *rn, blockIdx.x == 0, img, red, aux, tile, lane);
    else
        gemm8_wave_loop<T, NR>(acc, Wt + ((size_t)tile * nKB + s0) * T::TILE_BYTES, A8 + (size_t)s0 * RD_A8_BLOCK_BYTES, nk, aux, tile, lane, lane * 16);
    double2 cs[PPT];
    float b1 = 0.f, b2 = 0.f;
    if (isQ || isK) {
#pragma unroll
        for (int i = 0; i < PPT; i++) cs[i] = e.cs[(size_t)(e.row0 + min((tid >> 4) + 4 * KW * i, M - 1)) * half + d1];
    }
    if (e.bias) b1 = e.bias[head * HD + d1], b2 = e.bias[head * HD + d2];
    gemm8_fold_waves<KW, 1, T::INT_ACC>(acc, lds);
    float *sums = lds; // [32 rows][33]: the tile's sums, row stride 33 words against bank conflicts; the fold is done with this memory
    if (kw == 0) {
        T::finish(acc, aux, A8, tile, lane);
#pragma unroll
        for (int r = 0; r < 16; r++) sums[((r >> 2) * 8 + (lane >> 5) * 4 + (r & 3)) * 33 + (lane & 31)] = acc[r];
    }
    __syncthreads();
    const int kvh = isK ? head - e.nH : head - e.nH - e.nKV;
#pragma unroll
    for (int i = 0; i < PPT; i++) {
        const int mr = (tid >> 4) + 4 * KW * i, m = e.row0 + mr;
        float x1 = sums[mr * 33 + pi], x2 = sums[mr * 33 + pi + 16];
        if (mr >= M) continue;
        if (e.bias) x1 = __fadd_rn(x1, b1), x2 = __fadd_rn(x2, b2);
        float o1 = x1, o2 = x2;
        if (isQ || isK) o1 = rope_first(x1, x2, cs[i].x, cs[i].y), o2 = rope_second(x1, x2, cs[i].x, cs[i].y);
        if (isQ) {
            float *dst = e.q + (size_t)m * e.nH * HD + (size_t)head * HD;
            dst[d1] = o1, dst[d2] = o2;
        } else {
            const int p = where[i] & 63;
            const size_t region = ((size_t)(where[i] >> 6) * e.nKV + kvh) * 64 * HD;
            uint16_t *dst = (isK ? e.Kp : e.Vp) + region;
            const int i1 = isK ? (HD == 128 ? k_elem_index<128>(p, d1) : k_elem_index<64>(p, d1)) : (HD == 128 ? v_elem_index<128>(p, d1) : v_elem_index<64>(p, d1));
            const int i2 = isK ? (HD == 128 ? k_elem_index<128>(p, d2) : k_elem_index<64>(p, d2)) : (HD == 128 ? v_elem_index<128>(p, d2) : v_elem_index<64>(p, d2));
            dst[i1] = f32_to_f16_half_up(o1), dst[i2] = f32_to_f16_half_up(o2);
        }
    }
}

#define RD_GEMM8_QKV_KERNEL(NAME, TRAITS, KW)                                                                                                          \
    extern "C" __global__ __launch_bounds__(64 * KW) void NAME(                                                                                        \
        const uint8_t *__restrict__ Wt, const void *__restrict__ aux, const uint8_t *__restrict__ A8, int N, int nKB, int M, float *__restrict__ q,     \
        uint16_t *__restrict__ Kp, uint16_t *__restrict__ Vp, const int *__restrict__ tables, int tabStride, const int *__restrict__ rowSlot,           \
        const int *__restrict__ rowPos, const double *__restrict__ cs, const float *__restrict__ bias, int nH, int nKV, int HD, size_t a8Stride) {      \
        __shared__ float lds[KW > 2 ? (KW - 1) * 1024 : 32 * 33];                                                                                      \
        const int row0 = 32 * (int)blockIdx.z; /* M-tile z: rows row0.. of the step, activations a8Stride bytes further on */                          \
        A8 += (size_t)blockIdx.z * a8Stride, M = min(32, M - row0);                                                                                    \
        QkvEpilogue e{q, Kp, Vp, tables, rowSlot, rowPos, (const double2 *)cs, bias, tabStride, nH, nKV, HD, row0};                                    \
        if (TRAITS::GEMV1 && M == 1)                                                                                                                   \
            gemm8_qkv_body<TRAITS, KW, 1>(Wt, aux, A8, N, nKB, M, e, lds);                                                                             \
        else if (M <= 8)                                                                                                                               \
            gemm8_qkv_body<TRAITS, KW, 4>(Wt, aux, A8, N, nKB, M, e, lds);                                                                             \
        else if (M <= 16)                                                                                                                              \
            gemm8_qkv_body<TRAITS, KW, 8>(Wt, aux, A8, N, nKB, M, e, lds);                                                                             \
        else                                                                                                                                           \
            gemm8_qkv_body<TRAITS, KW, 16>(Wt, aux, A8, N, nKB, M, e, lds);                                                                            \
    }
// A one-row step's q|k|v projection with the norm-and-quantize kernel that feeds it folded in (see rd_k_gemm8_q4k_gateup_norm1):
// the same bits as rd_k_add_rmsnorm_quant followed by the kernel above, in one launch less. Grid (N/32), block KW waves.
#define RD_GEMM8_QKV_NORM1_KERNEL(NAME, TRAITS, KW)                                                                                                    \
    extern "C" __global__ __launch_bounds__(64 * KW) void NAME(                                                                                        \
        const uint8_t *__restrict__ Wt, const void *__restrict__ aux, int N, int nKB, float *__restrict__ q, uint16_t *__restrict__ Kp,                \
        uint16_t *__restrict__ Vp, const int *__restrict__ tables, int tabStride, const int *__restrict__ rowSlot, const int *__restrict__ rowPos,      \
        const double *__restrict__ cs, const float *__restrict__ bias, int nH, int nKV, int HD, const float *__restrict__ hIn, float *__restrict__ hOut, \
        const float *__restrict__ P, int splits, const float *__restrict__ w, float eps, int H) {                                                      \
        __shared__ float lds[KW > 2 ? (KW - 1) * 1024 : 32 * 33];                                                                                      \
        __shared__ __align__(16) uint8_t img[16 * RD_ROW0_KB_BYTES];                                                                                   \
        __shared__ double red[16];                                                                                                                     \
        QkvEpilogue e{q, Kp, Vp, tables, rowSlot, rowPos, (const double2 *)cs, bias, tabStride, nH, nKV, HD, 0};                                       \
        const Row0Norm rn{hIn, hOut, P, w, splits, H, eps};                                                                                            \
        gemm8_qkv_body<TRAITS, KW, 1, true>(Wt, aux, nullptr, N, nKB, 1, e, lds, &rn, img, red);                                                       \
    }
RD_GEMM8_QKV_NORM1_KERNEL(rd_k_gemm8_q4k_qkv_norm1_kw2, Q4K8Traits, 2)
RD_GEMM8_QKV_NORM1_KERNEL(rd_k_gemm8_q4k_qkv_norm1_kw4, Q4K8Traits, 4)
RD_GEMM8_QKV_NORM1_KERNEL(rd_k_gemm8_q4k_qkv_norm1_kw8, Q4K8Traits, 8)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_q4k_qkv_kw2, Q4K8Traits, 2)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_q4k_qkv_kw4, Q4K8Traits, 4)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_q4k_qkv_kw8, Q4K8Traits, 8)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_w8a8_qkv_kw2, W8A8Traits8, 2)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_w8a8_qkv_kw4, W8A8Traits8, 4)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_w8a8_qkv_kw8, W8A8Traits8, 8)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_w4a8_qkv_kw2, W4A8Traits8, 2)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_w4a8_qkv_kw4, W4A8Traits8, 4)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_w4a8_qkv_kw8, W4A8Traits8, 8)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_w8a8r_qkv_kw2, W8A8RowTraits8, 2)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_w8a8r_qkv_kw4, W8A8RowTraits8, 4)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_w8a8r_qkv_kw8, W8A8RowTraits8, 8)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_w4a8r_qkv_kw2, W4A8RowTraits8, 2)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_w4a8r_qkv_kw4, W4A8RowTraits8, 4)
RD_GEMM8_QKV_KERNEL(rd_k_gemm8_w4a8r_qkv_kw8, W4A8RowTraits8, 8)
