// device.h — the device object behind rd_device: the HIP module, its kernels, one stream, and small helpers.
#pragma once
#include "../../../include/rocmdecode.h"
#include "hipdyn.h"
#include <stdarg.h>
#include <stdio.h>
#include <algorithm>
#include <string>
#include <vector>

void rd_set_error(const char *fmt, ...);
bool rd_hip_ok(const HipApi *hip, hipError_t e, const char *what);
#define HIPCHK(call)                                                      \
    do {                                                                  \
        if (!rd_hip_ok(d->hip, d->hip->call, #call)) return RD_ERR_HIP;   \
    } while (0)

// sizes shared with the kernels (goinfer_amd/csrc/kernels/common.h)
constexpr size_t Q4K_TILE_BYTES = 4608;
constexpr size_t A8_BLOCK_BYTES = 10240; // one A8 activation block: 256 elements x 32 rows (gemm8.h)
inline size_t a8_bytes(int K) { return (size_t)((K + 255) / 256) * A8_BLOCK_BYTES; }
enum { PANEL_A8 = 3, PANEL_ROW8 = 4 }; // = RD_PANEL_* of the kernels
// dynamic LDS of the experts' GEMM kernels: four rows of K elements (codes, scales, sums) + their exchange area
inline unsigned moe_gemv_lds(int K) { return (unsigned)(4 * ((K + 255) / 256) * 320 + 1024); }
constexpr int MOE_GEMV_MAX_K = 12288; // 4 rows x 48 blocks x 320 B + 1 KB = 61 KB of LDS
// grid.x of rd_k_moe_gemv_w4a8 (moe.h): a wave streams about four 256-element blocks, as whole tiles of 32 weight rows (measured on
// the Qwen3-MoE down projection, K = 768: one tile a wave 27 us a launch, two tiles 30 us, four 41 us)
inline unsigned moe_gemv_grid(int N, int K) {
    int per = std::max(1, 4 / ((K + 255) / 256));
    if (const char *e = getenv("ROCMDECODE_MOE_TILES")) per = std::max(1, atoi(e));
    return (unsigned)((N / 32 + 4 * per - 1) / (4 * per));
}

struct Kernels {
    hipFunction_t dequant_q4k, quant_act, quant_act_row, reduce_splits, add_rmsnorm_quant, swiglu_quant, swiglu_quant_row;
    hipFunction_t unpack_act8, unpanel_a8, retile_q4k8, retile_w8a8_8, retile_w4a8_8;
    // [lane: 0 q4k, 1 w8a8, 2 w4a8 (per-32 activations), 3 w8a8, 4 w4a8 with one activation scale per row, 5 q5k, 6 q6k][waves per tile 2, 4, 8]
    hipFunction_t gemm8[7][3];
    hipFunction_t gemm8_qkv[7][3]; // the q|k|v projection with RoPE and the KV store in its epilogue, indexed like gemm8
    // Q4_K for passes of more than 32 rows: four M-tiles against each decoded weight tile (_g2: a second group of waves halves the K
    // ranges, for grids of few weight tiles)
    hipFunction_t gemm8_q4k_rows, gemm8_q4k_rows_g2, gemm8_q4k_rows_gateup, gemm8_q4k_rows_gateup_gelu, gemm8_q4k_rows_qkv, gemm8_q4k_rows_qkv_g2;
    hipFunction_t gemm8_q5k_rows, gemm8_q5k_rows_g2, gemm8_q6k_rows, gemm8_q6k_rows_g2; // the plain many-row kernel over Q5_K / Q6_K tiles
    hipFunction_t gemm8_q4k_gateup_norm1, gemm8_q4k_gateup_gelu_norm1, gemm8_q4k_qkv_norm1[3]; // a one-row step's projections with the norm folded in
    hipFunction_t gemm8_q4k_gateup, gemm8_q4k_gateup_gelu, add_one, moe_gemv_w4a8, moe_gemv_w4a8r, moe_gemv_w4a8r_f32in, moe_gemv_w4a8_gateup, moe_gemv_w4a8r_gateup, retile_w4a8_gv, rope_table;
    hipFunction_t dequant_q5k, retile_q5k, dequant_q6k, retile_q6k;
    hipFunction_t kv_store, kv_read, qkv_rope_store, attn_partial, attn_partial_wide, attn_combine, attn_combine_quant;
    hipFunction_t kv_store_i8, qkv_rope_store_i8, attn_partial_i8, attn_partial_rows, attn_partial_rows_i8, attn_partial_deep, attn_partial_deep_i8, topk_rows, topk_hist, topk_pick, topk_finish;
    hipFunction_t rmsnorm, rope, argmax_rows, argmax_final, matmul_f32, moe_route, moe_swiglu_quant, moe_swiglu_quant_row, moe_fold, embed_rows, copy16, fill_f16, fill_f32, issue_mfma_i8, issue_mfma_f32, issue_valu, issue_all;
};

struct rd_device {
    const HipApi *hip = nullptr;
    int ordinal = 0;
    hipModule_t module = nullptr;
    hipStream_t stream = nullptr;
    Kernels k{};
    std::vector<void *> owned; // device allocations freed at close

    // the same with `lds` bytes of dynamic shared memory
    template <typename... A> int launch_lds(hipFunction_t f, unsigned gx, unsigned gy, unsigned gz, unsigned bx, unsigned lds, A... a) {
        void *args[] = {(void *)&a...};
        hipError_t e = hip->ModuleLaunchKernel(f, gx, gy, gz, bx, 1, 1, lds, stream, args, nullptr);
        return rd_hip_ok(hip, e, "hipModuleLaunchKernel") ? RD_OK : RD_ERR_HIP;
    }
    template <typename... A> int launch(hipFunction_t f, unsigned gx, unsigned gy, unsigned gz, unsigned bx, A... a) {
        void *args[] = {(void *)&a...};
        hipError_t e = hip->ModuleLaunchKernel(f, gx, gy, gz, bx, 1, 1, 0, stream, args, nullptr);
        return rd_hip_ok(hip, e, "hipModuleLaunchKernel") ? RD_OK : RD_ERR_HIP;
    }
    // HIP's current device belongs to the calling thread, and a caller's threads come and go (a Go program's goroutines move
    // between OS threads): every call that allocates, copies or starts a step makes this device current first.
    int use();
    int alloc(void **p, size_t n);
    void release(void *p);
    int h2d(void *dst, const void *src, size_t n);
    int d2h(void *dst, const void *src, size_t n);
    int sync();
};

// A device buffer that frees itself (for the call-scoped temporaries of the kernel-level entry points).
struct DevBuf {
    rd_device *d;
    void *p = nullptr;
    explicit DevBuf(rd_device *dev) : d(dev) {}
    ~DevBuf() {
        if (p) d->release(p);
    }
    int alloc(size_t n) { return d->alloc(&p, n ? n : 16); }
    template <typename T> T *as() { return (T *)p; }
};

// block sizes that match the code object's launch bounds: the fused gate|up kernel (two tiles x two waves), the expert kernels
// (two tiles x two waves)
constexpr unsigned GATEUP_THREADS = 256, MOE_THREADS = 256;
// grid.z of the experts' gate|up kernels: an expert's passes of four rows run side by side in this many layers of blocks (one
// layer while no expert can have a fifth row; ROCMDECODE_MOE_PASS_LAYERS overrides, for measurement). Measured on the
// Qwen3-MoE-shape step of 16 rows: two layers take the gate|up launches from 1.86 to 1.77 ms a step; the down projection's
// launches, whose blocks are fewer and longer, lose by it (1.32 to 1.36 ms) and keep one layer.
inline unsigned moe_pass_layers(int T) {
    if (const char *e = getenv("ROCMDECODE_MOE_PASS_LAYERS")) return (unsigned)std::max(1, std::min(8, atoi(e)));
    return T > 4 ? 2u : 1u;
}

// How many 64-position KV blocks one attention work item covers for a sequence of nb blocks: every (sequence, kv head) is
// cut into pieces. The cut depends on the sequence's own length only, never on what else is in the
// batch: the partial results are merged in piece order, so this is what keeps a row computed in a batch bit-identical to
// the same row computed alone.
constexpr int ATTN_PIECES = 16; // = RD_ATTN_PIECES of the combine kernels: pieces they fold per round
// Blocks per item: a sixteenth of the sequence, but at most ATTN_MAX_CHUNK blocks (512 keys), so that a sequence of more than 128
// blocks is cut into more than 16 items and even a lone long sequence spreads over the chip. (A cap of four blocks serves a
// lone 8k-token sequence better, 18 against 29 us per layer, but costs the 64-sequence attention benchmark 5 %.)
constexpr int ATTN_MAX_CHUNK = 8;
inline int attn_chunk_blocks(int nb) { return std::min((nb + ATTN_PIECES - 1) / ATTN_PIECES, ATTN_MAX_CHUNK); }
// the most items one (row, kv head) of a sequence of up to nb blocks is cut into
inline int attn_max_pieces(int nb) { return std::max(ATTN_PIECES, (nb + ATTN_MAX_CHUNK - 1) / ATTN_MAX_CHUNK); }

// One attention work item: blocks [b0,b1) of one kv head of one sequence, for the step's row `row` — or, from the grouping
// builder, for rows row..row+n-1 with n in the high 16 bits of kvh; one wave each.
struct AttnItemH {
    int row, kvh, b0, b1;
};
constexpr int ATTN_RANGE_INTS = 3; // per (row, kv head): first item, one past the last, the row's place among its items' positions
// A work list of at most this many items (one per SIMD of the chip) runs the attention kernels that keep two units in flight
// per wave: with so few waves nothing else hides a wave's memory latency. Same results bit for bit.
constexpr int ATTN_DEEP_MAX_ITEMS = 1024;
// A step's work list is launched padded to a multiple of this many items (one per compute unit) with items whose row is -1
constexpr int ATTN_LIST_PAD = 256;
// Waves a block of rd_k_attn_partial_wide (= RD_ATTN_BLOCK_WAVES of the kernels), which takes the lists of at least
// ATTN_WIDE_MIN_ITEMS items (two waves for every SIMD of the chip)
constexpr int ATTN_BLOCK_WAVES = 4, ATTN_WIDE_MIN_ITEMS = 2048;
static_assert(ATTN_LIST_PAD % ATTN_BLOCK_WAVES == 0, "a padded list fills whole blocks");
// Pads a work list for launching (whole blocks whatever kernel takes it).
inline void attn_pad_items(std::vector<AttnItemH> &items) {
    items.resize((items.size() + ATTN_LIST_PAD - 1) / ATTN_LIST_PAD * ATTN_LIST_PAD, AttnItemH{-1, 0, 0, 0});
}
// The attention kernel for a (padded) work list of n_items and the waves it runs a block: grid = n_items / waves, block = 64 * waves.
struct AttnLaunch {
    hipFunction_t f;
    unsigned waves;
};
AttnLaunch attn_partial_kernel(const struct rd_device *d, bool i8, bool grouped, size_t n_items);
const char *attn_partial_kernel_name(const struct rd_device *d, hipFunction_t f);
constexpr int TOPK_MAX = 1024; // = RD_TOPK_MAX of the top-K kernels
constexpr int TOPK_CAP = 4096, TOPK_BINS = 2048, TOPK_CHUNK = 16384; // = RD_TOPK_CAP, RD_TOPK_BINS, RD_TOPK_CHUNK
// Scratch of the top-K over `rows` rows of width V (device memory the caller owns): per-chunk histograms and maxima, candidate
// counts (zero between calls), candidate lists, per-chunk shares of Z, and 1/T per row.
struct TopkScratch {
    int *ghist = nullptr, *ccount = nullptr, *cand_i = nullptr;
    unsigned *gmax = nullptr;
    float *cand_v = nullptr, *invT = nullptr;
    double *zpart = nullptr;
};
int topk_scratch_alloc(struct rd_device *d, int rows, int V, TopkScratch *s); // allocates and zeroes; the caller releases the seven buffers
// Rows of logits (device, [rows][V]) to ids, vals ([rows][k]) and z ([rows], may be null) on the device. invT: scalar used when
// rowsInvT is false, else s.invT holds one per row. Wide rows go over the chip in three launches, narrow ones take one block each.
int launch_topk(struct rd_device *d, const float *logits, int rows, int V, int k, float invT, bool rowsInvT, const TopkScratch &s, int *ids,
                float *vals, double *z);
constexpr int ATTN_TILE_ROWS = 16; // head rows of the attention MFMA tile: an item holds at most 16 / (heads per kv head) positions
// The attention work list of a step: items of the longest sequences first (the grid is dispatched in index order, so the
// short items fill the tail), and ranges[3*(row*n_kv+kvh)..] as above.
// slot == nullptr: one position per item. Otherwise consecutive rows of one slot whose lengths ascend by one and need the same
// number of blocks (so their cuts coincide) share items, up to 16/G of them; returns true if any item holds more than one
// position, in which case the step runs the kernels that read the high bits of kvh and write 16 head rows per item.
// window > 0: a sliding-window layer's list: a row's items cover only the blocks from position len-window on, and rows share
// items only when those first blocks coincide as well.
bool build_attn_worklist(const int *len, const int *slot, int G, int rows, int n_kv, std::vector<AttnItemH> &items, std::vector<int> &ranges,
                         int window = 0);

// split-K plan of one GEMM launch
struct GemmPlan {
    int splits;     // grid.y
    int kbPerSplit; // K-blocks (blocks of 256, or 128 for Q6_K) per split
    int kw = 0;     // int8-MFMA kinds: waves per weight tile inside a block, each on its own K range (2, 4 or 8)
};
// act_group 0 (one activation scale per row): one split, since the row's scale multiplies the finished sum inside the kernel
GemmPlan plan_gemm(int kind, int N, int nKB, int act_group = 32);

// Weight matrix resident on the device in its GEMM tiling.
struct DevWeight {
    int kind = -1; // 0 q4k, 1 w8a8, 2 w4a8, 3 q5k, 4 q6k, 5 a group of weights of different kinds stacked row-wise (parts)
    int N = 0, K = 0;
    void *tiled = nullptr;  // re-tiled codes
    void *scales = nullptr; // w8a8: f32[N]
    // goinfer's WeightMat.ActQuantGroup() for the int8 / int4 kinds: 32 = activations quantized per group of 32 (its q4k mode), 0 =
    // one scale per row (its int8 / int4 modes; the only lane its staged QuantBackend hooks serve). K-quants are always 32.
    int act_group = 32;
    std::vector<DevWeight> parts; // kind 5: the members, each of one kind, rows [col0[i], col0[i] + parts[i].N) of the group
    std::vector<int> col0;
};
enum { WKIND_GROUP = 5 };

int upload_q4k(rd_device *d, const void *blocks, int N, int K, DevWeight *w);
int upload_q5k(rd_device *d, const void *blocks, int N, int K, DevWeight *w);
int upload_q6k(rd_device *d, const void *blocks, int N, int K, DevWeight *w);
int upload_w8a8(rd_device *d, const int8_t *q, const float *row_scale, int N, int K, DevWeight *w, int act_group = 32);
int upload_w4a8(rd_device *d, const uint8_t *nib, const uint16_t *s16, int N, int K, DevWeight *w, bool expert = false, int act_group = 32);
// The activation quantizer a weight's GEMM expects of its producer: 32 or 0 (see DevWeight::act_group); a group's members agree.
int act_group_for(const DevWeight &w);
// index into Kernels::gemm8 / gemm8_qkv
inline int gemm8_lane(const DevWeight &w) { return w.kind >= 3 ? w.kind + 2 : (w.act_group == 0 && w.kind >= 1 ? w.kind + 2 : w.kind); }
// x f32 [M][K] on the device -> the panels of `kind`, quantized per 32 (act_group 32) or per row (0). M <= 32.
int launch_quant_act(rd_device *d, const float *x, int M, int K, int kind, int act_group, void *Xp);
void free_weight(rd_device *d, DevWeight *w);
// P[splits][32][N] = panels(Xp) . W^T ; returns the plan used
// ldP: floats between rows of P (0 = w.N); splits > 0 forces the split count (trailing splits that get no K-block store zeros),
// which lets weights of different kinds write side by side into one partial-sum buffer.
// Q4_K, int8 and int4-g32 weights go through the int8-MFMA kernels over A8 activation blocks (gemm8.h), Q5_K and Q6_K through
// the f16-MFMA kernels over f16 panels (kquant.h). kw > 0 forces the waves per tile of the int8-MFMA kinds.
// resid != NULL (int8-MFMA kinds, one split): the sums are added to resid[m][n] (row stride ldP) in place and nothing goes to P.
// M > 32 (int8-MFMA kinds only): further M-tiles of 32 rows, xpStride bytes / pStride floats apart, ride in the same launch (grid.z).
int launch_gemm(rd_device *d, const DevWeight &w, const void *Xp, float *P, int M, GemmPlan *plan, int ldP = 0, int splits = 0, int kw = 0,
                float *resid = nullptr, size_t xpStride = 0, size_t pStride = 0);
inline bool is_gemm8_kind(int kind) { return kind >= 0 && kind <= 4; } // every kind but a group: all run the int8-MFMA kernels
// Up to 128 rows as M-tiles of 32: M-tile mt reads its panels at Xp + mt*xpStride (bytes) and writes its partial sums at
// P + mt*pStride (floats), each laid out as launch_gemm's; the int8 kernels take the M-tiles as grid.z of one launch, the others one
// launch per M-tile. Either way a row is the same row whatever pass it rides in.
constexpr int GEMM_WIDE_ROWS = 512;
// the many-row Q4_K kernels: whether a grid of `blocks` blocks of four waves takes the second group of waves (under two waves per SIMD otherwise)
bool rows_gemm_enabled();
// rows from which a pass takes them: with one or two M-tiles half of a block's waves would idle, and the 32-row kernel over the
// M-tiles is faster (9.3 against 7.9 ms a step at 64 rows of the Llama-3-8B shape; 14.0 against 14.7 at 128)
constexpr int ROWS_GEMM_MIN_ROWS = 65;
void topk_static_prepare_device(int ordinal); // ops.cc: opens the allocation-free top-K's library and looks its scratch up for this device
inline bool rows_gemm_two_groups(size_t blocks) { return blocks < 2u * 256u; }
int launch_gemm_wide(rd_device *d, const DevWeight &w, const void *Xp, size_t xpStride, float *P, size_t pStride, int M, GemmPlan *plan, int ldP = 0,
                     int splits = 0, int kw = 0);
size_t panel_bytes_for(const DevWeight &w);
int panel_kind_for(const DevWeight &w);
// K-blocks of a weight: 256 elements (an A8 block, a Q5_K super-block), 128 for Q6_K's half super-blocks. The int8-MFMA kinds pad K up to whole blocks with zeros.
inline int kblock_of(int) { return 256; }
inline int kblocks_for(const DevWeight &w) { return (w.K + kblock_of(w.kind) - 1) / kblock_of(w.kind); }
