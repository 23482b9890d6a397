// moe.h — expert-major MoE FFN (goinfer decoder/mlp.go:630-726 moeMLPBatchWith; CUDA analogue backend/cuda/moe_rows.cu).
// A step has at most 32 tokens. Every touched expert's weights are streamed once per GEMM for the rows routed to it (a second
// time only past four rows); rankOf[token][expert] (from rd_k_moe_route) is the map from tokens to experts and ranks.
#pragma once
#include "act.h"
#include "gemm8.h"

// The expert grid row `row` works on, or -1 (uniform over the block; every thread must call it).
__device__ __forceinline__ int moe_block_expert(const unsigned *__restrict__ activeBits, const signed char *__restrict__ rankOf, int nE, int T, int row) {
    int e = row;
    if (activeBits) {
        int y = row;
        for (int w = 0; w < (nE + 31) >> 5; w++) {
            unsigned b = activeBits[w];
            const int c = __popc(b);
            if (y < c) {
                for (int i = 0; i < y; i++) b &= b - 1; // drop the y lowest set bits
                return w * 32 + __ffs((int)b) - 1;
            }
            y -= c;
        }
        return -1;
    }
    int mine = ((int)threadIdx.x < T && rankOf[(size_t)threadIdx.x * nE + e] >= 0) ? 1 : 0;
    return __syncthreads_or(mine) ? e : -1;
}

// The experts' GEMMs run on the vector ALU, not on the matrix cores. A decode step gives an expert one to three rows (16 tokens x
// top-8 over 128 experts), and a 32-row MFMA tile pays for all 32: the per-group fold alone (a convert and an fma per output and
// group) costs more than the whole product does with v_dot4_i32_i8 over the rows that exist. Per wave: 32 weight rows x its share
// of K; lane (row n, parity h) takes the groups 2p+h of every 256-element block, so one lane forms a group's whole int32 dot
// (eight dot4 over the signed values nib-8) and folds it as the reference does (facc = fma(idot, aS*wS, facc)); the two
// parities' sums are added at the end (even groups + odd groups), then the KW waves' in wave order. The expert's rows come four at
// a time from LDS (codes, scales, sums; gathered by token); an expert with more than four rows takes another pass over its
// weights. Arithmetic: exact int32 dot per group, f32 fold; the same for any number of rows in the step.
//
// Weight tile (rd_k_retile_w4a8_gv), 4608 B per 32 rows x 256 k like the MFMA kernels' tile: 32 headers of 16 B (the row's eight
// group scales, f16), then four planes [64 lanes][16 B]: plane p, lane (row r, parity h), byte b = element b of group 2p+h in
// the low nibble and element 16+b in the high nibble, each as the two's-complement nibble of its value nib-8 (= nib ^ 8): moved
// to the top of a byte it is the int8 16*(nib-8), so a dot4 over such bytes is 16 times the group's signed dot, exactly, and
// the 1/16 rides in the scale (a power of two).
extern "C" __global__ __launch_bounds__(320) void rd_k_retile_w4a8_gv(const uint8_t *__restrict__ nib, const uint16_t *__restrict__ s16,
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
            const int klo = kb * 256 + (2 * p + h) * 32 + b, khi = klo + 16;
            const int lo = klo < K ? (row[klo >> 1] >> (4 * (klo & 1))) & 15 : 8, hi = khi < K ? (row[khi >> 1] >> (4 * (khi & 1))) & 15 : 8;
            by[b] = (uint8_t)((lo ^ 8) | ((hi ^ 8) << 4));
        }
        __builtin_memcpy(&v, by, 16);
    }
    *(uint4_t *)(dst + (size_t)t * 16) = v;
}

// The tokens of expert e in ascending order are its rows 0, 1, ...: *src = the token that is row (lane & 31), or -1 past the
// last. Returns the number of rows. Every lane of the wave must call it.
__device__ __forceinline__ int moe_expert_rows(const signed char *__restrict__ rankOf, int nE, int T, int e, int lane, int *src) {
    const bool mine = lane < T && rankOf[(size_t)lane * nE + e] >= 0;
    const uint32_t mk = (uint32_t)__ballot(mine);
    uint32_t rest = mk;
    for (int i = 0; i < (lane & 31); i++) rest &= rest - 1; // drop the lane & 31 lowest tokens
    *src = rest ? __ffs((int)rest) - 1 : -1;
    return __popc(mk);
}

constexpr int GV_ROWS = 4; // rows of an expert worked on per pass over its weights (two: 6.32 against 5.91 ms a Qwen3-MoE-shape step)
// LDS of a pass: the rows' codes [GV_ROWS][Kpad] (Kpad = K up to whole 256-blocks, zero-filled), then their scales [GV_ROWS][Kpad/32].
__device__ __forceinline__ size_t gv_lds_bytes(int nKB) { return (size_t)GV_ROWS * nKB * (256 + 32); }

// Stage the rows of a pass into LDS. X: ROW8 activations of K elements; row j of the pass is X's row rowOf[j] (>= 0) or all
// zeros. All threads of the block call it with the same rowOf; the caller synchronizes.
__device__ __forceinline__ void gv_stage(uint8_t *lds, const uint8_t *__restrict__ X, int K, int nKB, const int (&rowOf)[GV_ROWS]) {
    const int Kpad = nKB * 256, nGp = nKB * 8, nG = K >> 5;
    float *ldsS = (float *)(lds + (size_t)GV_ROWS * Kpad);
    for (int i = threadIdx.x; i < GV_ROWS * (Kpad >> 4); i += blockDim.x) {
        const int j = i / (Kpad >> 4), c = i - j * (Kpad >> 4), row = j == 0 ? rowOf[0] : (j == 1 ? rowOf[1] : (j == 2 ? rowOf[2] : rowOf[3]));
        uint4_t v = {0u, 0u, 0u, 0u};
        if (row >= 0 && c * 16 < K) v = *(const uint4_t *)(X + (size_t)row * K + c * 16);
        *(uint4_t *)(lds + (size_t)j * Kpad + c * 16) = v;
    }
    for (int i = threadIdx.x; i < GV_ROWS * nGp; i += blockDim.x) {
        const int j = i / nGp, g = i - j * nGp, row = j == 0 ? rowOf[0] : (j == 1 ? rowOf[1] : (j == 2 ? rowOf[2] : rowOf[3]));
        ldsS[i] = row >= 0 && g < nG ? *(const float *)(X + row8_scales(K) + ((size_t)row * nG + g) * 4) : 0.f;
    }
}

// The same from rows that are still f32 (an expert's silu(gate)*up rows, XF [32][K]) and their maxima (rowMax, the bits of max |x|
// accumulated by the kernel that wrote them): the per-row quantizer (linalg.QuantizeRowInt8: scale maxabs/127, codes
// round-half-away) runs as the rows are staged, so the rows never exist as codes in memory and SwiGLU needs no launch of its own.
__device__ __forceinline__ void gv_stage_f32(uint8_t *lds, const float *__restrict__ XF, const unsigned *__restrict__ rowMax, int K, int nKB,
                                             const int (&rowOf)[GV_ROWS]) {
    const int Kpad = nKB * 256, nGp = nKB * 8;
    float *ldsS = (float *)(lds + (size_t)GV_ROWS * Kpad);
    for (int i = threadIdx.x; i < GV_ROWS * (Kpad >> 2); i += blockDim.x) {
        const int j = i / (Kpad >> 2), c = i - j * (Kpad >> 2), row = j == 0 ? rowOf[0] : (j == 1 ? rowOf[1] : (j == 2 ? rowOf[2] : rowOf[3]));
        uint32_t codes = 0u;
        if (row >= 0 && c * 4 < K) {
            const float inv = 1.f / row_scale_of(__uint_as_float(rowMax[row]));
            const float4_t v = *(const float4_t *)(XF + (size_t)row * K + c * 4);
            const int c0 = (int)fminf(127.f, fmaxf(-127.f, roundf(__fmul_rn(v.x, inv)))), c1 = (int)fminf(127.f, fmaxf(-127.f, roundf(__fmul_rn(v.y, inv))));
            const int c2 = (int)fminf(127.f, fmaxf(-127.f, roundf(__fmul_rn(v.z, inv)))), c3 = (int)fminf(127.f, fmaxf(-127.f, roundf(__fmul_rn(v.w, inv))));
            codes = (uint32_t)(c0 & 255) | ((uint32_t)(c1 & 255) << 8) | ((uint32_t)(c2 & 255) << 16) | ((uint32_t)(c3 & 255) << 24);
        }
        *(uint32_t *)(lds + (size_t)j * Kpad + c * 4) = codes;
    }
    for (int i = threadIdx.x; i < GV_ROWS * nGp; i += blockDim.x) {
        const int j = i / nGp, row = j == 0 ? rowOf[0] : (j == 1 ? rowOf[1] : (j == 2 ? rowOf[2] : rowOf[3]));
        ldsS[i] = row >= 0 ? row_scale_of(__uint_as_float(rowMax[row])) : 0.f;
    }
}

// One 256-element block of the wave's tile against the R staged rows (R the same on every lane: the rows past it are skipped
// by a scalar branch, one body of code for any R). kb: the block's index in K.
// ROW: the rows carry one activation scale each (ActQuantGroup 0): the fold takes the weight's group scale alone, as the reference's
// expert kernels do (backend/cuda/moe_rows.cu:60-75, moe.cu:116-173), and the caller multiplies the finished sum by the row's scale.
template <bool ROW>
__device__ __forceinline__ void gv_block(float (&facc)[GV_ROWS], const Q4K8Tile &w, const uint8_t *lds, int nKB, int kb, int h, int R) {
    const int Kpad = nKB * 256, nGp = nKB * 8;
    const float *ldsS = (const float *)(lds + (size_t)GV_ROWS * Kpad);
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const uint32_t wd = w.hdr[p];
        const float ws = f16_bits_to_f32((uint16_t)(h ? wd >> 16 : wd & 0xffffu));
        const uint4_t raw = w.q[p];
        uint32_t lo[4], hi[4]; // bytes 16 * (nib - 8): elements 0..15 and 16..31 of the group
#pragma unroll
        for (int i = 0; i < 4; i++) lo[i] = (raw[i] << 4) & 0xF0F0F0F0u, hi[i] = raw[i] & 0xF0F0F0F0u;
        const int g = kb * 8 + 2 * p + h;
#pragma unroll
        for (int j = 0; j < GV_ROWS; j++) {
            if (j >= R) continue;
            const uint4_t a0 = *(const uint4_t *)(lds + (size_t)j * Kpad + g * 32), a1 = *(const uint4_t *)(lds + (size_t)j * Kpad + g * 32 + 16);
            int idot = 0;
#pragma unroll
            for (int i = 0; i < 4; i++) idot = __builtin_amdgcn_sdot4((int)lo[i], (int)a0[i], idot, false);
#pragma unroll
            for (int i = 0; i < 4; i++) idot = __builtin_amdgcn_sdot4((int)hi[i], (int)a1[i], idot, false);
            // idot = 16 * sum (nib-8) * a, a multiple of 16: the shift is exact
            facc[j] = __builtin_fmaf((float)(idot >> 4), ROW ? ws : __fmul_rn(ldsS[j * nGp + g], ws), facc[j]);
        }
    }
}

// A wave's stream of weight tiles for one pass: nTiles tiles of nKB 256-element blocks each, one after the other with three
// blocks in flight the whole way (the next tile's first blocks are asked for while the current tile's last are worked on), so
// the wave pays its start-up once. tileOff(q): byte offset of tile q's first block inside the descriptor; past the last tile
// the loads go out of the descriptor's range and are answered with zeros. At the end of tile q: epi(q, facc), with facc[j] the
// tile row's sum for staged row j on the lanes of both parities (parity 0's groups + parity 1's).
struct GvTiles {
    Q4K8Tile w[3];
};
template <class TileOff>
__device__ __forceinline__ int gv_offset(int u, int nTiles, int nKB, TileOff tileOff) {
    const int q = u / nKB;
    return u < nTiles * nKB ? tileOff(q) + (u - q * nKB) * 4608 : 0x7ff00000;
}
// the stream's first three blocks, asked for before the pass's rows are staged so that the two waits overlap
template <class TileOff>
__device__ __forceinline__ void gv_first(GvTiles &t, rd_rsrc_t wr, int nTiles, TileOff tileOff, int nKB, int lane) {
#pragma unroll
    for (int i = 0; i < 3; i++) Q4K8Traits::load(t.w[i], wr, gv_offset(i, nTiles, nKB, tileOff), lane);
}
template <bool ROW, class TileOff, class Epi>
__device__ __forceinline__ void gv_stream(GvTiles &t, rd_rsrc_t wr, int nTiles, TileOff tileOff, int nKB, const uint8_t *lds, int lane, int R, Epi epi) {
    const int U = nTiles * nKB, h = lane >> 5;
    auto off = [&](int u) { return gv_offset(u, nTiles, nKB, tileOff); };
    float facc[GV_ROWS];
#pragma unroll
    for (int j = 0; j < GV_ROWS; j++) facc[j] = 0.f;
    Q4K8Tile(&w)[3] = t.w;
    int q = 0, kb = 0;
    for (int u = 0; u < U; u += 3) {
#pragma unroll
        for (int i = 0; i < 3; i++) {
            if (u + i < U) gv_block<ROW>(facc, w[i], lds, nKB, kb, h, R);
            Q4K8Traits::load(w[i], wr, off(u + i + 3), lane); // unconditional: the count of loads in flight stays exact
            if (u + i < U && ++kb == nKB) {
#pragma unroll
                for (int j = 0; j < GV_ROWS; j++) {
                    const float other = __shfl_xor(facc[j], 32, 64);
                    facc[j] = h ? __fadd_rn(other, facc[j]) : __fadd_rn(facc[j], other);
                }
                epi(q, facc);
#pragma unroll
                for (int j = 0; j < GV_ROWS; j++) facc[j] = 0.f;
                kb = 0, q++;
            }
        }
    }
}

// out[(token*k + rank)][N] = X . W_e^T for the experts that have at least one token. Grid (gx, nE), block 256: four waves, each
// streaming ceil(N / 32 / (4 gx)) consecutive tiles of 32 weight rows over the whole K (the launch picks gx: few tiles per wave
// for a deep K, several for a shallow one, so that a wave has enough blocks to stream to pay for its start-up). X: ROW8 activations of K elements;
// xStride: bytes between the experts' own activations, whose rows are the expert's tokens in ascending order (what
// rd_k_moe_gemv_w4a8_gateup and rd_k_moe_swiglu_quant write), or 0: all experts read the step's rows (row = token) and gather theirs.
// activeBits (may be NULL): the bitmap of experts with a token. Row y of the grid then works on the y-th expert whose bit is set,
// and the rows past the last one exit: the blocks with work are the first in dispatch order, which spreads them evenly over
// the XCDs and CUs (blocks are handed out round-robin; idle ones scattered among them skew that). Without the bitmap row y is
// expert y, and exits when no token chose it. Dynamic LDS: gv_lds_bytes(nKB).
// F32IN (with ROW): X is the experts' f32 rows [expert][32][K] and rowMax their maxima [expert][32]; they are quantized per row as staged.
template <bool ROW, bool F32IN = false>
__device__ __forceinline__ void moe_gemv_body(const uint8_t *__restrict__ Wt, size_t wStride, const uint8_t *__restrict__ X, size_t xStride,
                                              float *__restrict__ out, int N, int K, int T, int k, const signed char *__restrict__ rankOf, int nE,
                                              const unsigned *__restrict__ activeBits, uint8_t *lds, const unsigned *__restrict__ rowMax = nullptr) {
    const int nKB = (K + 255) >> 8;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    // xStride != 0: every expert reads activations of its own, so all blocks of an expert are placed on one XCD (blocks go to the
    // eight XCDs round-robin in linear order) and its activations are pulled into one L2 instead of eight.
    int bx = blockIdx.x, row = blockIdx.y;
    if (xStride != 0 && (gridDim.y & 7) == 0) {
        const int gx = gridDim.x, L = row * gx + bx, j = L >> 3;
        row = (j / gx) * 8 + (L & 7), bx = j % gx;
    }
    const int e = moe_block_expert(activeBits, rankOf, nE, T, row);
    if (e < 0) return;
    Wt += (size_t)e * wStride, X += (size_t)e * xStride;
    const int perWave = ((N >> 5) + 4 * (int)gridDim.x - 1) / (4 * (int)gridDim.x);
    const int tile0 = (bx * 4 + wave) * perWave, nTiles = max(0, min(perWave, (N >> 5) - tile0));
    const rd_rsrc_t wr = make_rsrc(Wt, (uint32_t)((N >> 5) * nKB * 4608));
    auto tileOff = [&](int q) { return (tile0 + q) * nKB * 4608; };
    GvTiles wt;
    // The passes of an expert with more than GV_ROWS rows are dealt over grid.z (pass p to layer p % gridDim.z) and run side by
    // side instead of one after the other; the layers past an expert's passes find nothing to do and leave.
    bool primed = blockIdx.z == 0;
    if (primed) gv_first(wt, wr, nTiles, tileOff, nKB, lane); // the weights need only the expert: asked for before its rows are looked up
    int src;
    const int rows = moe_expert_rows(rankOf, nE, T, e, lane, &src);
    for (int r0 = (int)blockIdx.z * GV_ROWS; r0 < rows; r0 += (int)gridDim.z * GV_ROWS) {
        const int R = min(GV_ROWS, rows - r0);
        int rowOf[GV_ROWS], tokOf[GV_ROWS]; // uniform: the pass's rows in X and their tokens (a lane is never asked for a token while it sits out a branch)
#pragma unroll
        for (int j = 0; j < GV_ROWS; j++) {
            tokOf[j] = __builtin_amdgcn_readlane(src, min(r0 + j, 31));
            rowOf[j] = r0 + j < rows ? (xStride == 0 ? tokOf[j] : r0 + j) : -1;
        }
        if (!primed) gv_first(wt, wr, nTiles, tileOff, nKB, lane);
        primed = false;
        __syncthreads(); // the previous pass is done with the staged rows
        if constexpr (F32IN)
            gv_stage_f32(lds, (const float *)X, rowMax + (size_t)e * 32, K, nKB, rowOf);
        else
            gv_stage(lds, X, K, nKB, rowOf);
        __syncthreads();
        float rowS[GV_ROWS]; // ROW: the staged rows' scales (every group slot of a row holds it)
#pragma unroll
        for (int j = 0; j < GV_ROWS; j++) rowS[j] = ROW ? ((const float *)(lds + (size_t)GV_ROWS * nKB * 256))[j * nKB * 8] : 1.f;
        gv_stream<ROW>(
            wt, wr, nTiles, tileOff, nKB, lds, lane, R, [&](int q, const float(&facc)[GV_ROWS]) {
                if (lane < 32) {
#pragma unroll
                    for (int j = 0; j < GV_ROWS; j++)
                        if (j < R)
                            out[((size_t)tokOf[j] * k + rankOf[(size_t)tokOf[j] * nE + e]) * N + (tile0 + q) * 32 + lane] =
                                ROW ? mul_rounded(facc[j], rowS[j]) : facc[j];
                }
            });
    }
}
extern "C" __global__ __launch_bounds__(256) void rd_k_moe_gemv_w4a8(const uint8_t *__restrict__ Wt, size_t wStride, const uint8_t *__restrict__ X,
                                                                      size_t xStride, float *__restrict__ out, int N, int K, int T, int k,
                                                                      const signed char *__restrict__ rankOf, int nE,
                                                                      const unsigned *__restrict__ activeBits) {
    extern __shared__ __align__(16) uint8_t lds[];
    moe_gemv_body<false>(Wt, wStride, X, xStride, out, N, K, T, k, rankOf, nE, activeBits, lds);
}
// The same over rows that carry one activation scale each (ActQuantGroup 0: the "int8 per-token activations" of the Qwen3-MoE benchmark configuration).
extern "C" __global__ __launch_bounds__(256) void rd_k_moe_gemv_w4a8r(const uint8_t *__restrict__ Wt, size_t wStride, const uint8_t *__restrict__ X,
                                                                       size_t xStride, float *__restrict__ out, int N, int K, int T, int k,
                                                                       const signed char *__restrict__ rankOf, int nE,
                                                                       const unsigned *__restrict__ activeBits) {
    extern __shared__ __align__(16) uint8_t lds[];
    moe_gemv_body<true>(Wt, wStride, X, xStride, out, N, K, T, k, rankOf, nE, activeBits, lds);
}
// The experts' down projection over rows still in f32 (what rd_k_moe_gemv_w4a8r_gateup leaves): XF [expert][32][K] f32 with the
// expert's tokens in ascending order as rows 0, 1, ..., rowMax [expert][32] the bits of each row's max |x|. The same values as
// rd_k_moe_swiglu_quant_row followed by rd_k_moe_gemv_w4a8r, bit for bit, in one launch less.
extern "C" __global__ __launch_bounds__(256) void rd_k_moe_gemv_w4a8r_f32in(const uint8_t *__restrict__ Wt, size_t wStride, const float *__restrict__ XF,
                                                                             const unsigned *__restrict__ rowMax, float *__restrict__ out, int N, int K,
                                                                             int T, int k, const signed char *__restrict__ rankOf, int nE,
                                                                             const unsigned *__restrict__ activeBits) {
    extern __shared__ __align__(16) uint8_t lds[];
    moe_gemv_body<true, true>(Wt, wStride, (const uint8_t *)XF, (size_t)32 * K * sizeof(float), out, N, K, T, k, rankOf, nE, activeBits, lds, rowMax);
}

// The experts' gate|up projection with SwiGLU and the per-32 quantization in its epilogue (same values as rd_k_moe_gemv_w4a8
// followed by rd_k_moe_swiglu_quant, bit for bit). Wt per expert: [gate rows; up rows] (2*I rows). Grid (ceil(I / 64), nE),
// block 256: waves 0 and 2 stream gate tiles 2x and 2x+1 over the whole K, waves 1 and 3 the matching up tiles; a gate wave
// leaves its sums in LDS and its up wave forms silu(gate) * up over the tile's 32 columns, which are one activation group,
// quantizes it and writes it as row r0+j of the expert's own ROW8 activations XE (I elements a row). X: the step's rows, ROW8,
// K elements. Dynamic LDS: gv_lds_bytes(nKB) + 1 KB.
// ROW: the step's rows carry one activation scale each and the output stays f32 — XF [expert][32][I] with the expert's tokens as
// rows 0, 1, ... and rowMax [expert][32] taking the bits of each row's max |silu(gate)*up| through atomicMax (zero on entry;
// non-negative floats order as their bits): the per-row quantizer needs the whole row, which no block of this kernel has, so it
// runs where the rows are staged next (rd_k_moe_gemv_w4a8r_f32in).
template <bool ROW>
__device__ __forceinline__ void moe_gateup_body(const uint8_t *__restrict__ Wt, size_t wStride, const uint8_t *__restrict__ X, uint8_t *__restrict__ XE,
                                                size_t xeStride, float *__restrict__ XF, unsigned *__restrict__ rowMax, int I, int K, int T,
                                                const signed char *__restrict__ rankOf, int nE, const unsigned *__restrict__ activeBits, uint8_t *dyn) {
    float *xch = (float *)dyn; // [2 pairs][GV_ROWS][32]: the gate waves' sums
    uint8_t *lds = dyn + 1024;
    const int nKB = (K + 255) >> 8;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int e = moe_block_expert(activeBits, rankOf, nE, T, blockIdx.y);
    if (e < 0) return;
    Wt += (size_t)e * wStride;
    if constexpr (!ROW) XE += (size_t)e * xeStride;
    const int nGate = I >> 5, pair = wave >> 1, isUp = wave & 1, t = blockIdx.x * 2 + pair, nTiles = t < nGate ? 1 : 0;
    const rd_rsrc_t wr = make_rsrc(Wt, (uint32_t)(2 * nGate * nKB * 4608));
    auto tileOff = [&](int) { return (isUp * nGate + t) * nKB * 4608; };
    GvTiles wt;
    bool primed = blockIdx.z == 0; // passes over grid.z as in moe_gemv_body
    if (primed) gv_first(wt, wr, nTiles, tileOff, nKB, lane); // the weights need only the expert: asked for before its rows are looked up
    int src;
    const int rows = moe_expert_rows(rankOf, nE, T, e, lane, &src);
    for (int r0 = (int)blockIdx.z * GV_ROWS; r0 < rows; r0 += (int)gridDim.z * GV_ROWS) {
        const int R = min(GV_ROWS, rows - r0);
        int rowOf[GV_ROWS];
#pragma unroll
        for (int j = 0; j < GV_ROWS; j++) {
            const int tok = __builtin_amdgcn_readlane(src, min(r0 + j, 31));
            rowOf[j] = r0 + j < rows ? tok : -1;
        }
        if (!primed) gv_first(wt, wr, nTiles, tileOff, nKB, lane);
        primed = false;
        __syncthreads(); // the previous pass is done with the staged rows and the exchanged sums
        gv_stage(lds, X, K, nKB, rowOf);
        __syncthreads();
        float sum[GV_ROWS] = {};
        gv_stream<ROW>(wt, wr, nTiles, tileOff, nKB, lds, lane, R, [&](int, const float(&facc)[GV_ROWS]) {
#pragma unroll
            for (int j = 0; j < GV_ROWS; j++) sum[j] = facc[j];
        });
        if constexpr (ROW) { // the row's scale multiplies the finished sum
#pragma unroll
            for (int j = 0; j < GV_ROWS; j++) sum[j] = mul_rounded(sum[j], ((const float *)(lds + (size_t)GV_ROWS * nKB * 256))[j * nKB * 8]);
        }
        if (!isUp && lane < 32) {
#pragma unroll
            for (int j = 0; j < GV_ROWS; j++) xch[(pair * GV_ROWS + j) * 32 + lane] = sum[j];
        }
        __syncthreads();
        if (isUp && nTiles) {
#pragma unroll
            for (int j = 0; j < GV_ROWS; j++)
                if (j < R) { // the same on every lane: both halves of the wave hold the row's 32 columns
                    const float act = __fmul_rn(silu_f64(xch[(pair * GV_ROWS + j) * 32 + (lane & 31)]), sum[j]);
                    if constexpr (ROW) {
                        const size_t row = (size_t)e * 32 + r0 + j;
                        if (lane < 32) XF[row * I + t * 32 + lane] = act;
                        const float ma = wave_max32(fabsf(act));
                        if (lane == 0) atomicMax(rowMax + row, __float_as_uint(ma));
                    } else {
                        const Quant1 qv = quant_one(act);
                        if (lane < 32) panel_store(XE, RD_PANEL_ROW8, r0 + j, t * 32 + lane, qv, I);
                    }
                }
        }
    }
}
extern "C" __global__ __launch_bounds__(256) void rd_k_moe_gemv_w4a8_gateup(const uint8_t *__restrict__ Wt, size_t wStride,
                                                                             const uint8_t *__restrict__ X, uint8_t *__restrict__ XE,
                                                                             size_t xeStride, int I, int K, int T,
                                                                             const signed char *__restrict__ rankOf, int nE,
                                                                             const unsigned *__restrict__ activeBits) {
    extern __shared__ __align__(16) uint8_t dyn[];
    moe_gateup_body<false>(Wt, wStride, X, XE, xeStride, nullptr, nullptr, I, K, T, rankOf, nE, activeBits, dyn);
}
extern "C" __global__ __launch_bounds__(256) void rd_k_moe_gemv_w4a8r_gateup(const uint8_t *__restrict__ Wt, size_t wStride,
                                                                              const uint8_t *__restrict__ X, float *__restrict__ XF,
                                                                              unsigned *__restrict__ rowMax, int I, int K, int T,
                                                                              const signed char *__restrict__ rankOf, int nE,
                                                                              const unsigned *__restrict__ activeBits) {
    extern __shared__ __align__(16) uint8_t dyn[];
    moe_gateup_body<true>(Wt, wStride, X, nullptr, 0, XF, rowMax, I, K, T, rankOf, nE, activeBits, dyn);
}

// gate/up rows [(token,rank)][2I] -> silu(gate)*up -> per-32 quantization -> the down-projection activations of that row's expert,
// at the token's place among the expert's tokens. Grid (ceil(I/256), T*k).
extern "C" __global__ __launch_bounds__(256) void rd_k_moe_swiglu_quant(const float *__restrict__ gu, const int *__restrict__ idx, int I, int k,
                                                                        uint8_t *__restrict__ XpE, size_t xpStride, const signed char *__restrict__ rankOf,
                                                                        int nE) {
    int row = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x, tok = row / k, e = idx[row];
    int t = 0; // tokens before this one that chose the same expert
    for (int i = 0; i < tok; i++) t += rankOf[(size_t)i * nE + e] >= 0;
    float a = 0.f;
    if (n < I) {
        float g = gu[(size_t)row * 2 * I + n], u = gu[(size_t)row * 2 * I + I + n];
        a = __fmul_rn(silu_f64(g), u);
    }
    const Quant1 q = quant_one(a);
    if (n < I) panel_store(XpE + (size_t)e * xpStride, RD_PANEL_ROW8, t, n, q, I);
}

// The same with one scale per row of I (ActQuantGroup 0; backend/cuda/moe_rows.cu glu_quant_rows): one block of 256 threads per
// (token, rank) row, four consecutive columns per thread and round, up to eight rounds (I <= 8192, I % 32 == 0) kept in registers
// between the row's maximum and its codes. Grid (T*k).
extern "C" __global__ __launch_bounds__(256) void rd_k_moe_swiglu_quant_row(const float *__restrict__ gu, const int *__restrict__ idx, int I, int k,
                                                                            uint8_t *__restrict__ XpE, size_t xpStride,
                                                                            const signed char *__restrict__ rankOf, int nE) {
    __shared__ float red[16];
    const int row = blockIdx.x, tok = row / k, e = idx[row], nv = I >> 2;
    int t = 0; // tokens before this one that chose the same expert
    for (int i = 0; i < tok; i++) t += rankOf[(size_t)i * nE + e] >= 0;
    float4_t a[8];
    float ma = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int q = threadIdx.x + i * 256;
        a[i] = (float4_t){0.f, 0.f, 0.f, 0.f};
        if (q >= nv) continue;
        const float4_t g = *(const float4_t *)(gu + (size_t)row * 2 * I + 4 * q), u = *(const float4_t *)(gu + (size_t)row * 2 * I + I + 4 * q);
#pragma unroll
        for (int c = 0; c < 4; c++) a[i][c] = __fmul_rn(silu_f64(g[c]), u[c]);
        ma = fmaxf(ma, fmaxf(fmaxf(fabsf(a[i].x), fabsf(a[i].y)), fmaxf(fabsf(a[i].z), fabsf(a[i].w))));
    }
    const float s = row_scale_of(block_max(ma, red));
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int q = threadIdx.x + i * 256;
        if (q >= nv) continue; // groups of 8 lanes are on or off together
        const Quant4 qq = quant_four_row(a[i].x, a[i].y, a[i].z, a[i].w, s);
        panel_store4(XpE + (size_t)e * xpStride, RD_PANEL_ROW8, t, 4 * q, qq, I);
    }
}

// out[t][:] = sum over ranks, in rank order, of wgt[t][rank] * down[(t,rank)][:]  (decoder/mlp.go:100-103, addScaled: mul then add).
extern "C" __global__ void rd_k_moe_fold(const float *__restrict__ dn, const float *__restrict__ wgt, float *__restrict__ out, int H, int k) {
    int t = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x;
    if (n >= H) return;
    float acc = 0.f;
    for (int r = 0; r < k; r++) acc = __fadd_rn(acc, mul_rounded(wgt[t * k + r], dn[((size_t)t * k + r) * H + n]));
    out[(size_t)t * H + n] = acc;
}
