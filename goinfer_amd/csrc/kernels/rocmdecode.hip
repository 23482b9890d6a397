// rocmdecode.hip — the single translation unit of the gfx950 code object (rocmdecode_gfx950.hsaco).
// Every entry point is an extern "C" __global__ so the host side (or a Go purego binding) finds it by name with
// hipModuleGetFunction.
#include "common.h"
#include "q4k.h"
#include "act.h"
#include "attn.h"
#include "gemm8.h"
#include "gemm8_rows.h"
#include "kquant.h"
#include "misc.h"
#include "moe.h"
#include "topk.h"

// Attention combine fused with the per-32 quantization that feeds the o-projection. Grid (nH, rows), block
// RD_ATTN_PIECES * HD/4; the first HD/4 threads (whole 8-lane quantization groups) finish the row.
extern "C" __global__ __launch_bounds__(512) void rd_k_attn_combine_quant(const float *__restrict__ part, const int *__restrict__ itemStart, int partRows,
                                                                           uint8_t *__restrict__ Xp, int kind, int nH, int nKV, int HD,
                                                                           size_t xpStride, const float *__restrict__ sinks) {
    __shared__ float lds[RD_ATTN_PIECES * (128 + 2)];
    const int head = blockIdx.x, m = blockIdx.y;
    float v[4];
    if (!attn_combine_block(part, itemStart, partRows, nH, nKV, HD, m, head, lds, v, sinks)) return;
    const Quant4 q = quant_four(v[0], v[1], v[2], v[3]);
    panel_store4(Xp + (size_t)(m >> 5) * xpStride, kind, m & 31, head * HD + threadIdx.x * 4, q); // M-tile m/32, row m%32
}
