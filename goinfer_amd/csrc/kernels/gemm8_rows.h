// gemm8_rows.h — the Q4_K projections for passes of more than two row tiles of 32 (65 to 512 rows: a prompt, a ragged step with a
// prompt chunk riding, a wide decode batch):
// goinfer's prompt-rate GEMM (backend/cuda/gemm_w4a8_mma.cu:57-188 keeps several row tiles of accumulators against one weight tile).
//
// A block owns one 32-row weight tile (and one K split) and four M-tiles of 32 batch rows, one per wave. Per super-block the four
// waves decode the tile once between them (wave p: the scales of sub-blocks 2p, 2p+1 and plane p's nibbles widened to the int8
// operands of v_mfma_i32_32x32x32_i8) into LDS, two buffers deep, and each wave multiplies the decoded tile with its own M-tile's
// A8 activations. What the 32-row kernels spend per M-tile on reading, unpacking and decoding weights is spent once per 128 rows.
//
// Same bits as the 32-row kernels: a wave walks the K ranges that the 32-row kernel deals to its KW waves one after the other,
// each range from a zero accumulator, and adds the finished ranges in ascending order, which is the order of gemm8_fold_waves;
// within a range the arithmetic is Q4K8Traits::mma<16>, operation for operation. A row's sums are those it gets alone.
//
// Where the grid has too few tiles to give every SIMD two waves, a block takes a second group of four waves (G = 2): the groups
// share the M-tiles and halve the K ranges between them (group 1 the upper half), each with its own decoded tiles. Group 1 leaves
// every finished range in LDS, and group 0 adds them after its own, still in ascending order.
#pragma once
#include "gemm8.h"

constexpr int RD_ROWS_MT = 4;    // M-tiles (waves of a group) per block
constexpr int RD_ROWS_PARTS = 4; // K ranges group 1 can leave (KW <= 8)

// What a weight format brings to the kernel: its tile's size, the size of the decoded tile in LDS, a wave's share of the raw tile
// (three 16-byte loads a lane), its share of the decoding, and the product of a decoded tile with an activation block.
struct RowsRaw {
    uint4_t hdr, q, x; // header bytes, the wave's nibble plane, the format's extra plane (fifth bits, high bit pairs) or nothing
};

// Q4_K (Q5 = false) and Q5_K (Q5 = true: the Q4_K tile followed by a plane of fifth bits, Q5K8Traits). Decoded tile: lo [4][64][16 B],
// hi [4][64][16 B] (the int8 operands of sub-blocks 2p and 2p+1), dsc [64][4] f32, ndm [64][4] f32.
template <bool Q5>
struct RowsQ45 {
    static constexpr int TB = Q5 ? 5632 : 4608, BUF = 4096 + 4096 + 1024 + 1024;
    // off: the tile's byte offset in the descriptor's range; plane: the wave's plane
    static __device__ __forceinline__ void load(RowsRaw &w, rd_rsrc_t r, int off, int plane, int lane) {
        w.hdr = buf_load16_nt(r, off + (lane & 31) * 16, 0);
        w.q = buf_load16_nt(r, off + 512 + plane * 1024 + lane * 16, 0);
        if constexpr (Q5) w.x = buf_load16_nt(r, off + 4608 + lane * 16, 0);
    }
    // wave p: the scales of sub-blocks 2p, 2p+1 (Q4K8Traits::decode's arithmetic) and plane p's nibbles (and fifth bits) widened
    static __device__ __forceinline__ void decode(uint8_t *buf, int p, int lane, const RowsRaw &w) {
        const uint32_t y = w.hdr.y, z = w.hdr.z, x = w.hdr.w, hx = w.hdr.x;
        half2_t dd;
        __builtin_memcpy(&dd, &hx, 4);
        const float d = (float)dd.x, dmin = (float)dd.y;
        const int h = lane >> 5;
        int sc, mn;
        if (p < 2) { // sub-blocks 0..3
            const int j8 = 8 * (2 * p + h);
            sc = (y >> j8) & 63, mn = (z >> j8) & 63;
        } else { // sub-blocks 4..7
            const int j8 = 8 * (2 * p - 4 + h);
            sc = ((x >> j8) & 15) | (((y >> (j8 + 6)) & 3) << 4), mn = ((x >> (j8 + 4)) & 15) | (((z >> (j8 + 6)) & 3) << 4);
        }
        uint4_t lo, hi;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            lo[i] = w.q[i] & 0x0F0F0F0Fu, hi[i] = (w.q[i] >> 4) & 0x0F0F0F0Fu;
            if constexpr (Q5) lo[i] |= ((w.x[i] >> (2 * p)) & 0x01010101u) << 4, hi[i] |= ((w.x[i] >> (2 * p + 1)) & 0x01010101u) << 4;
        }
        *(uint4_t *)(buf + (p * 64 + lane) * 16) = lo;
        *(uint4_t *)(buf + 4096 + (p * 64 + lane) * 16) = hi;
        *(float *)(buf + 8192 + (lane * 4 + p) * 4) = __fmul_rn(d, (float)sc);
        *(float *)(buf + 9216 + (lane * 4 + p) * 4) = -__fmul_rn(dmin, (float)mn);
    }
    // acc += the decoded tile times the activation block a: Q4K8Traits::mma<16> (Q5K8Traits' is the same) with its operands from LDS
    static __device__ __forceinline__ void mma(float16_t &acc, const uint8_t *buf, int lane, const A8Regs &a) {
        const f32x32_t zero32 = {0.f};
        const i32x16_t zero16 = {0};
        const float4_t dsc = *(const float4_t *)(buf + 8192 + lane * 16), ndm = *(const float4_t *)(buf + 9216 + lane * 16);
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const uint4_t lo = *(const uint4_t *)(buf + (p * 64 + lane) * 16), hi = *(const uint4_t *)(buf + 4096 + (p * 64 + lane) * 16);
            const f32x32_t s2 = __builtin_amdgcn_mfma_f32_32x32x1f32(a.as[p], dsc[p], zero32, 0, 0, 0);
            const i32x16_t d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[2 * p]), as_i32x4(lo), zero16, 0, 0, 0);
            const i32x16_t d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[2 * p + 1]), as_i32x4(hi), zero16, 0, 0, 0);
            RD_FOLD(acc, d0, s2, 0, 16)
            RD_FOLD(acc, d1, s2, 16, 16)
        }
#pragma unroll
        for (int p = 0; p < 4; p++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.asum[p], ndm[p], acc, 0, 0, 0);
    }
};

// Q6_K (the 7168-byte tile of Q6K8Traits). Decoded tile: cl [8][64][16 B], ch [8][64][16 B] (group g's int8 operand with the upper /
// the lower lane half's elements zeroed: one product per 16-element sub-block), dscale [64 lanes][8] f32 (d/4 * the lane's sub-block
// scale of group g). Wave p decodes groups 2p and 2p+1.
struct RowsQ6 {
    static constexpr int TB = 7168, BUF = 8192 + 8192 + 2048;
    static __device__ __forceinline__ void load(RowsRaw &w, rd_rsrc_t r, int off, int plane, int lane) {
        w.hdr = buf_load16_nt(r, off + lane * 16, 0);
        w.q = buf_load16_nt(r, off + 1024 + plane * 1024 + lane * 16, 0);
        w.x = buf_load16_nt(r, off + 5120 + (plane >> 1) * 1024 + lane * 16, 0); // groups 2p, 2p+1 sit in high-bit plane p / 2
    }
    static __device__ __forceinline__ void decode(uint8_t *buf, int p, int lane, const RowsRaw &w) {
        const bool upper = lane >= 32;
        const float d = f16_bits_to_f32((uint16_t)(w.hdr.z & 0xffffu)) * 0.25f; // the codes come out as 4 * (q - 32)
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int g = 2 * p + j;
            const int sci = (int)((g < 4 ? w.hdr.x : w.hdr.y) << (24 - 8 * (g & 3))) >> 24;
            const uint32_t hw = (g & 3) == 0 ? w.x.x : ((g & 3) == 1 ? w.x.y : ((g & 3) == 2 ? w.x.z : w.x.w));
            uint4_t cl, ch;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const uint32_t nib = j ? (w.q[i] >> 2) & 0x3C3C3C3Cu : (w.q[i] << 2) & 0x3C3C3C3Cu;
                const uint32_t c = nib | ((hw << (6 - 2 * i)) & 0xC0C0C0C0u);
                cl[i] = upper ? 0u : c, ch[i] = upper ? c : 0u;
            }
            *(uint4_t *)(buf + (g * 64 + lane) * 16) = cl;
            *(uint4_t *)(buf + 8192 + (g * 64 + lane) * 16) = ch;
            *(float *)(buf + 16384 + (lane * 8 + g) * 4) = __fmul_rn(d, (float)sci);
        }
    }
    // Q6K8Traits::mma<16> with its operands from LDS
    static __device__ __forceinline__ void mma(float16_t &acc, const uint8_t *buf, int lane, const A8Regs &a) {
        const f32x32_t zero32 = {0.f};
        const i32x16_t zero16 = {0};
        const float4_t s03 = *(const float4_t *)(buf + 16384 + lane * 32), s47 = *(const float4_t *)(buf + 16384 + lane * 32 + 16);
#pragma unroll
        for (int g = 0; g < 8; g++) {
            const int p = g >> 1;
            float a_lo, a_hi;
            halves_f(a.as[p], a_lo, a_hi);
            const f32x32_t s2 = __builtin_amdgcn_mfma_f32_32x32x1f32((g & 1) ? a_hi : a_lo, g < 4 ? s03[g & 3] : s47[g & 3], zero32, 0, 0, 0);
            const uint4_t cl = *(const uint4_t *)(buf + (g * 64 + lane) * 16), ch = *(const uint4_t *)(buf + 8192 + (g * 64 + lane) * 16);
            const i32x16_t d0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[g]), as_i32x4(cl), zero16, 0, 0, 0);
            const i32x16_t d1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(as_i32x4(a.c[g]), as_i32x4(ch), zero16, 0, 0, 0);
            RD_FOLD(acc, d0, s2, 0, 16)
            RD_FOLD(acc, d1, s2, 16, 16)
        }
    }
};

template <class K> constexpr int rows_lds_bytes(int G) { return G * 2 * K::BUF + (G > 1 ? RD_ROWS_MT * RD_ROWS_PARTS * 4096 : 0); }

// The sums of NT weight tiles (one after the other: a gate tile and its up tile) over the split's super-blocks [0, nkb) for this
// wave's M-tile. wt[i]: tile i's first super-block of the split; a8: the M-tile's first activation block of the split (NULL: an
// M-tile past the pass's rows, which still takes its part in the decoding); per: super-blocks per K range and kw: ranges (the
// 32-row kernel's waves per tile). Every wave of the block calls it; the totals are valid in group 0 (waves 0..3).
template <int NT, int G, class K = RowsQ45<false>>
__device__ __forceinline__ void rows_core(float16_t (&total)[NT], const uint8_t *const (&wt)[NT], const uint8_t *__restrict__ a8, int nkb, int per, int kw,
                                          uint8_t *lds) {
    static_assert(G == 1 || NT == 1, "range groups are for single tiles");
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int g = G > 1 ? wave >> 2 : 0, plane = wave & 3; // the wave's group, and its M-tile = the plane it decodes
    constexpr int AB = RD_A8_BLOCK_BYTES, TB = K::TB, BUF = K::BUF;
    const int span = G > 1 ? (kw / G) * per : nkb;                      // super-blocks per group
    const int kbA = min(nkb, g * span), nk = min(nkb, kbA + span) - kbA; // this group's
    const int n = NT * nk, nLoop = NT * min(nkb, span);                 // steps of this group, and of group 0 (the longest)
    rd_rsrc_t wr[NT];
#pragma unroll
    for (int i = 0; i < NT; i++) wr[i] = make_rsrc(wt[i] + (size_t)kbA * TB, (uint32_t)nk * TB);
    const rd_rsrc_t ar = make_rsrc(a8 ? a8 + (size_t)kbA * AB : nullptr, a8 ? (uint32_t)nk * AB : 0u);
    uint8_t *bufs = lds + g * 2 * BUF;
    float4_t *parts = (float4_t *)(lds + G * 2 * BUF) + (size_t)plane * RD_ROWS_PARTS * 256; // [range][4][64 lanes] of this M-tile
    const int aoff = lane * 16;
    auto raw_load = [&](int s, RowsRaw &w) {
        int i = 0, kb = s;
        if (NT > 1 && s >= nk) i = 1, kb = s - nk;
        if (s >= n) kb = nk; // past the end: outside the range, zeros and no traffic
        K::load(w, (NT > 1 && i == 1) ? wr[NT - 1] : wr[0], kb * TB, plane, lane);
    };
    float16_t cur;
#pragma unroll
    for (int i = 0; i < NT; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) total[i][r] = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++) cur[r] = 0.f;
    if (nLoop <= 0) return;
    // One step: the next step's tile is decoded into the other buffer (its readers finished with it before the barrier that ended
    // the previous step), then this step's product; a finished K range joins the sum, the first as it is, the others added in
    // ascending order. The activation registers are refilled for the step two ahead as soon as the product has read them, so the
    // wait for them sits a whole step later (a0 serves the even steps, a1 the odd ones; a second tile reads the same blocks again).
    RowsRaw r0 = {}, r1 = {}; // the raw shares of the tiles one and two steps ahead
    auto step = [&](int s, A8Regs &a) {
        K::decode(bufs + ((s + 1) & 1) * BUF, plane, lane, r0);
        r0 = r1;
        raw_load(s + 3, r1);
        if (s < n && a8) { // (a wave whose M-tile lies past the pass's rows only decodes)
            const int kb = (NT > 1 && s >= nk) ? s - nk : s;
            K::mma(cur, bufs + (s & 1) * BUF, lane, a);
            {
                int kn = s + 2; // the step that reads these registers next
                if (NT > 1 && kn >= nk && kn < n) kn -= nk;
                else if (kn >= n) kn = nk; // none: outside the range
                a8_load(a, ar, kn * AB + aoff);
            }
            __builtin_amdgcn_sched_barrier(0); // the refill is issued here, not sunk to where its registers are next read
            if (((kb + 1) % per) == 0 || kb + 1 == nk) {
                const int li = kb / per; // the range's index within the group
                if (g == 0) {
                    const int i = (NT > 1 && s >= nk) ? 1 : 0;
#pragma unroll
                    for (int t = 0; t < NT; t++)
                        if (t == i) {
#pragma unroll
                            for (int r = 0; r < 16; r++) total[t][r] = li == 0 ? cur[r] : __fadd_rn(total[t][r], cur[r]);
                        }
                } else {
#pragma unroll
                    for (int q = 0; q < 4; q++) parts[(li * 4 + q) * 64 + lane] = (float4_t){cur[4 * q], cur[4 * q + 1], cur[4 * q + 2], cur[4 * q + 3]};
                }
#pragma unroll
                for (int r = 0; r < 16; r++) cur[r] = 0.f;
            }
        }
        __syncthreads();
    };
    A8Regs a0, a1;
    raw_load(0, r0);
    a8_load(a0, ar, aoff);
    raw_load(1, r1);
    a8_load(a1, ar, ((NT > 1 && nk == 1) ? 0 : (n > 1 ? 1 : nk)) * AB + aoff);
    K::decode(bufs, plane, lane, r0);
    r0 = r1;
    raw_load(2, r1);
    __syncthreads();
    for (int s = 0; s < nLoop; s += 2) {
        step(s, a0);
        if (s + 1 < nLoop) step(s + 1, a1);
    }
    if (G > 1 && g == 0) { // group 1's ranges, ascending (the last step's barrier put them in LDS)
        const int kbB = min(nkb, span);
        for (int li = 0; kbB + li * per < min(nkb, 2 * span); li++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const float4_t v = parts[(li * 4 + q) * 64 + lane];
                total[0][4 * q] = __fadd_rn(total[0][4 * q], v.x), total[0][4 * q + 1] = __fadd_rn(total[0][4 * q + 1], v.y);
                total[0][4 * q + 2] = __fadd_rn(total[0][4 * q + 2], v.z), total[0][4 * q + 3] = __fadd_rn(total[0][4 * q + 3], v.w);
            }
    }
}

// ---------------- plain projection ----------------
// Arguments as RD_GEMM8_KERNEL's plus kw, the 32-row kernel's waves per tile (it fixes the K ranges).
// Grid (N/32, splits, ceil(M/128)), block 256 * G.
template <int G, class K>
__device__ __forceinline__ void rows_plain_body(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ A8, float *__restrict__ P, int N, int nKB,
                                                int kbPerSplit, int kw, int M, int ldP, float *__restrict__ resid, size_t a8Stride, size_t pStride,
                                                uint8_t *lds) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int tile = blockIdx.x, split = blockIdx.y, mt = blockIdx.z * RD_ROWS_MT + (wave & 3);
    const int kb0 = split * kbPerSplit, kb1 = min(nKB, kb0 + kbPerSplit), nkb = max(kb1 - kb0, 0);
    const int per = max(1, (nkb + kw - 1) / kw);
    const int Mt = min(32, M - 32 * mt); // this wave's M-tile's rows
    float16_t total[1];
    const uint8_t *const wt[1] = {Wt + ((size_t)tile * nKB + kb0) * K::TB};
    rows_core<1, G, K>(total, wt, Mt > 0 ? A8 + (size_t)mt * a8Stride + (size_t)kb0 * RD_A8_BLOCK_BYTES : nullptr, nkb, per, kw, lds);
    if (Mt <= 0 || wave >= 4) return;
    const int n = tile * 32 + (lane & 31);
    if (resid) {
        float *rs = resid + (size_t)mt * 32 * ldP;
        float old[16];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            old[r] = rs[(size_t)min(m, Mt - 1) * ldP + n];
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            if (m < Mt) rs[(size_t)m * ldP + n] = __fadd_rn(old[r], total[0][r]);
        }
        return;
    }
    float *out = P + (size_t)mt * pStride + (size_t)split * 32 * ldP + n;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (m < Mt) out[(size_t)m * ldP] = total[0][r];
    }
}
#define RD_ROWS_PLAIN_KERNEL(NAME, G, K)                                                                                                        \
    extern "C" __global__ __launch_bounds__(256 * G) void NAME(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ A8, float *__restrict__ P, \
                                                               int N, int nKB, int kbPerSplit, int kw, int M, int ldP, float *__restrict__ resid,     \
                                                               size_t a8Stride, size_t pStride) {                                                     \
        __shared__ __attribute__((aligned(16))) uint8_t lds[rows_lds_bytes<K>(G)];                                                             \
        rows_plain_body<G, K>(Wt, A8, P, N, nKB, kbPerSplit, kw, M, ldP, resid, a8Stride, pStride, lds);                                          \
    }
RD_ROWS_PLAIN_KERNEL(rd_k_gemm8_q4k_rows, 1, RowsQ45<false>)
RD_ROWS_PLAIN_KERNEL(rd_k_gemm8_q4k_rows_g2, 2, RowsQ45<false>)
// Q5_K and Q6_K tensors (a Q4_K_M file keeps some of its projections in them): the same kernel over their tiles
RD_ROWS_PLAIN_KERNEL(rd_k_gemm8_q5k_rows, 1, RowsQ45<true>)
RD_ROWS_PLAIN_KERNEL(rd_k_gemm8_q5k_rows_g2, 2, RowsQ45<true>)
RD_ROWS_PLAIN_KERNEL(rd_k_gemm8_q6k_rows, 1, RowsQ6)
RD_ROWS_PLAIN_KERNEL(rd_k_gemm8_q6k_rows_g2, 2, RowsQ6)

// ---------------- fused gate|up projection + SwiGLU + per-32 quantization (rd_k_gemm8_q4k_gateup for more than 32 rows) ----------------
// Grid (I/32, 1, ceil(M/128)), block 256: a wave takes the gate tile and then the up tile of its M-tile over K (two K ranges each,
// as the 32-row kernel's two waves per tile), and has both finished tiles in registers in accumulator order, where a half-wave
// holds the 32 columns of one batch row: one activation group of the down projection, quantized where it sits.
template <int ACT>
__device__ __forceinline__ void rows_gateup_body(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ A8, uint8_t *__restrict__ XpOut, int I, int nKB,
                                                 int M, size_t a8Stride, size_t outStride, uint8_t *lds) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int t = blockIdx.x, nGate = I >> 5, mt = blockIdx.z * RD_ROWS_MT + wave;
    const int per = max(1, (nKB + 1) / 2), Mt = min(32, M - 32 * mt);
    float16_t total[2];
    const uint8_t *const wt[2] = {Wt + (size_t)t * nKB * 4608, Wt + (size_t)(nGate + t) * nKB * 4608};
    rows_core<2, 1>(total, wt, Mt > 0 ? A8 + (size_t)mt * a8Stride : nullptr, nKB, per, 2, lds);
    if (Mt <= 0) return;
    uint8_t *out = XpOut + (size_t)mt * outStride;
    const int n = t * 32 + (lane & 31);
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int m = (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        const float a = __fmul_rn(gate_act(total[0][r], ACT), total[1][r]);
        const Quant1 q = quant_one(a);
        // four neighbouring lanes hold four consecutive elements of the row: their codes leave as one word
        const int c = q.code & 255;
        const uint32_t word = (uint32_t)dpp_i<0x00>(c) | ((uint32_t)dpp_i<0x55>(c) << 8) | ((uint32_t)dpp_i<0xAA>(c) << 16) | ((uint32_t)dpp_i<0xFF>(c) << 24);
        if (m < Mt && (lane & 3) == 0) a8_store4(out, m, n, word, q.sc, q.gsum);
    }
}
#define RD_ROWS_GATEUP_KERNEL(NAME, ACT)                                                                                                            \
    extern "C" __global__ __launch_bounds__(256) void NAME(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ A8, uint8_t *__restrict__ XpOut, \
                                                           int I, int nKB, int M, size_t a8Stride, size_t outStride) {                             \
        __shared__ __attribute__((aligned(16))) uint8_t lds[rows_lds_bytes<RowsQ45<false>>(1)];                                                                     \
        rows_gateup_body<ACT>(Wt, A8, XpOut, I, nKB, M, a8Stride, outStride, lds);                                                                  \
    }
RD_ROWS_GATEUP_KERNEL(rd_k_gemm8_q4k_rows_gateup, 0)
RD_ROWS_GATEUP_KERNEL(rd_k_gemm8_q4k_rows_gateup_gelu, 1)

// ---------------- q|k|v projection with bias, RoPE and the KV store in its epilogue (rd_k_gemm8_q4k_qkv_kw* for more than 32 rows) ----------------
// Grid (N/32, 1, ceil(M/128)), block 256 * G; kw: the 32-row kernel's waves per tile. A wave of group 0 finishes its M-tile: the
// tile's sums go through the wave's own LDS square and its lanes take the 32 rows x 16 rotation pairs, eight pairs each.
template <int G>
__device__ __forceinline__ void rows_qkv_body(const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ A8, int N, int nKB, int kw, int M, const QkvEpilogue &e,
                                              size_t a8Stride, uint8_t *lds) {
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const int tile = blockIdx.x, mt = blockIdx.z * RD_ROWS_MT + (wave & 3);
    const int per = max(1, (nKB + kw - 1) / kw), Mt = min(32, M - 32 * mt);
    float16_t total[1];
    const uint8_t *const wt[1] = {Wt + (size_t)tile * nKB * 4608};
    rows_core<1, G>(total, wt, Mt > 0 ? A8 + (size_t)mt * a8Stride : nullptr, nKB, per, kw, lds);
    __syncthreads(); // every wave is done with the decoded tiles: the memory now takes the finished sums
    if (Mt <= 0 || wave >= 4) return;
    const int HD = e.HD, half = HD >> 1, head = (tile * 32) / HD, j = ((tile * 32) % HD) >> 5;
    const bool isQ = head < e.nH, isK = !isQ && head < e.nH + e.nKV;
    const int kvh = isK ? head - e.nH : head - e.nH - e.nKV;
    const int row0 = 32 * mt;
    float *sums = (float *)lds + wave * (32 * 33); // [32 rows][33]
#pragma unroll
    for (int r = 0; r < 16; r++) sums[((r >> 2) * 8 + (lane >> 5) * 4 + (r & 3)) * 33 + (lane & 31)] = total[0][r];
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_s_waitcnt(0xc07f); // lgkmcnt(0): the wave's own writes have landed before its lanes read them back
    const int pi = lane & 15, d1 = 16 * j + pi, d2 = half + d1; // this lane's pair: elements d1, d2 of the head, columns pi, pi + 16 of the tile
    float b1 = 0.f, b2 = 0.f;
    if (e.bias) b1 = e.bias[head * HD + d1], b2 = e.bias[head * HD + d2];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int mr = (lane >> 4) + 4 * i, m = row0 + mr;
        if (mr >= Mt) continue;
        float x1 = sums[mr * 33 + pi], x2 = sums[mr * 33 + pi + 16];
        if (e.bias) x1 = __fadd_rn(x1, b1), x2 = __fadd_rn(x2, b2);
        float o1 = x1, o2 = x2;
        if (isQ || isK) {
            const double2 cs = e.cs[(size_t)m * half + d1];
            o1 = rope_first(x1, x2, cs.x, cs.y), o2 = rope_second(x1, x2, cs.x, cs.y);
        }
        if (isQ) {
            float *dst = e.q + (size_t)m * e.nH * HD + (size_t)head * HD;
            dst[d1] = o1, dst[d2] = o2;
        } else {
            const int pos = e.rowPos[m], p = pos & 63;
            const int blk = e.tables[(size_t)e.rowSlot[m] * e.tabStride + (pos >> 6)];
            const size_t region = ((size_t)blk * e.nKV + kvh) * 64 * HD;
            uint16_t *dst = (isK ? e.Kp : e.Vp) + region;
            const int i1 = isK ? (HD == 128 ? k_elem_index<128>(p, d1) : k_elem_index<64>(p, d1)) : (HD == 128 ? v_elem_index<128>(p, d1) : v_elem_index<64>(p, d1));
            const int i2 = isK ? (HD == 128 ? k_elem_index<128>(p, d2) : k_elem_index<64>(p, d2)) : (HD == 128 ? v_elem_index<128>(p, d2) : v_elem_index<64>(p, d2));
            dst[i1] = f32_to_f16_half_up(o1), dst[i2] = f32_to_f16_half_up(o2);
        }
    }
}
#define RD_ROWS_QKV_KERNEL(NAME, G)                                                                                                                    \
    extern "C" __global__ __launch_bounds__(256 * G) void NAME(                                                                                        \
        const uint8_t *__restrict__ Wt, const uint8_t *__restrict__ A8, int N, int nKB, int kw, int M, float *__restrict__ q, uint16_t *__restrict__ Kp, \
        uint16_t *__restrict__ Vp, const int *__restrict__ tables, int tabStride, const int *__restrict__ rowSlot, const int *__restrict__ rowPos,      \
        const double *__restrict__ cs, const float *__restrict__ bias, int nH, int nKV, int HD, size_t a8Stride) {                                      \
        __shared__ __attribute__((aligned(16))) uint8_t lds[rows_lds_bytes<RowsQ45<false>>(G)];                                                        \
        static_assert(rows_lds_bytes<RowsQ45<false>>(G) >= 4 * 32 * 33 * 4, "the epilogue's squares fit the decode buffers");                                          \
        QkvEpilogue e{q, Kp, Vp, tables, rowSlot, rowPos, (const double2 *)cs, bias, tabStride, nH, nKV, HD, 0};                                       \
        rows_qkv_body<G>(Wt, A8, N, nKB, kw, M, e, a8Stride, lds);                                                                                     \
    }
RD_ROWS_QKV_KERNEL(rd_k_gemm8_q4k_rows_qkv, 1)
RD_ROWS_QKV_KERNEL(rd_k_gemm8_q4k_rows_qkv_g2, 2)
