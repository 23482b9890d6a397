// model.h — the resident decoder behind rd_model: weights in their GEMM tilings, the paged f16 KV pool, step scratch.
#pragma once
#include "device.h"
#include <map>
#include <vector>

// kernel classes of one decode step, for per-class timing
enum {
    KC_GEMM_QKV = 0, KC_ROPE_STORE, KC_ATTN_PARTIAL, KC_ATTN_COMBINE, KC_GEMM_O, KC_ADD_NORM, KC_GEMM_GATEUP, KC_SWIGLU, KC_GEMM_DOWN,
    KC_GEMM_HEAD, KC_ARGMAX, KC_MOE_ROUTER, KC_MOE_GEMM, KC_MOE_GEMM_DOWN, KC_MOE_GLUE, KC_COUNT
};

struct PendingMat { // a projection uploaded but not yet fused with its siblings (q|k|v, gate|up)
    int kind = -1, N = 0, K = 0;
    int act_group = 32; // int8 / int4 kinds: WeightMat.ActQuantGroup() (32, or 0 = one activation scale per row)
    std::vector<uint8_t> data;
    std::vector<uint8_t> scales;
};

struct LayerW {
    DevWeight qkv, o, gateup, down;
    PendingMat pend[RD_PROJ_COUNT];
    float *attn_norm = nullptr, *ffn_norm = nullptr, *q_norm = nullptr, *k_norm = nullptr;
    float *post_attn_norm = nullptr, *post_ffn_norm = nullptr; // optional: Gemma 2's norms of a branch's output before the residual add
    float *qkv_bias = nullptr; // optional: q bias, k bias, v bias end to end
    float *router_bias = nullptr; // optional [nE]: e_score_correction_bias (selection only)
    float *sinks = nullptr;       // optional [nH]: attention sinks
    int window = 0;               // > 0: sliding-window layer
    // MoE
    float *router = nullptr;           // [nE][hidden] f32
    void *exp_gateup = nullptr;        // [nE] stacked tiled W4A8, each 2*expert_inter rows x hidden
    void *exp_down = nullptr;          // [nE] stacked tiled W4A8, each hidden rows x expert_inter
    std::vector<char> exp_have;        // [nE*3]
    uint16_t *Kp = nullptr, *Vp = nullptr; // KV pool of this layer (binary16, or int8 codes when the model's kv_type says so)
    float *Ksc = nullptr, *Vsc = nullptr;  // int8 pool: one scale per (block, kv head, position)
};

struct StepTimer {
    bool on = false;
    std::vector<hipEvent_t> ev; // pairs
    std::vector<int> cls;
};

struct rd_model {
    rd_device *d = nullptr;
    rd_model_desc desc{};
    std::vector<double> inv_freq;
    double *inv_freq_dev = nullptr;
    double *rope_cs = nullptr; // [max_rows][head_dim/2] (cos, sin) of the step's RoPE angles, written once per step
    std::vector<LayerW> layers;
    DevWeight head;
    PendingMat head_pend;
    float *final_norm = nullptr;
    signed char *embed_q = nullptr; // optional device copy of the int8 embedding table (device-side greedy chain)
    float *embed_scale = nullptr;
    bool finalized = false;
    // router variant (decoder/mlp.go:130-228): sigmoid scoring, routed scaling factor, group-limited selection
    int router_sigmoid = 0, n_group = 0, topk_group = 0;
    float router_scale = 0.f;
    int window = 0; // the one window length the model's sliding-window layers share (0: none has one)
    int upload_act_group = 32; // what rd_model_set_act_group last set: the ActQuantGroup of the int8 / int4 uploads that follow
    int exp_act_group = -1;    // the experts' (one value for the model; -1 until the first expert tensor arrives)
    float *attn_out = nullptr; // [max_rows][n_heads*head_dim] f32: the attention output ahead of a per-row quantizer (allocated when an o projection takes per-row activations)
    int norm_add_one = 0, act = 0; // (1 + w) norm weights; the gated FFN's activation (RD_ACT_*)
    float final_softcap = 0.f;     // > 0: logits become cap * tanh(logit / cap)
    float logit_mul = 0.f;         // not 0 or 1: logits are multiplied by it after the softcap (f32(1 / LogitScale))
    bool ones_added = false;       // the (1 + w) pass over the norm weights has run
    bool bench_skip_attn = false;  // measurement only: the step leaves out its attention launches (its results are then meaningless)
    // The launches of a step as a captured HIP graph, replayed while steps keep one key (see step_run in model.cc)
    struct StepGraph {
        bool enabled = true;
        hipGraph_t graph = nullptr;
        hipGraphExec_t exec = nullptr;
        std::vector<long> key, prev_key;
        long captures = 0, replays = 0;
    } graph;

    // KV
    int slots = 0, ctx_cap = 0, blocks_per_slot = 0;
    int *tables = nullptr; // [slots][blocks_per_slot]
    std::vector<int> slot_len;

    // step scratch (device)
    float *h2 = nullptr; // a one-row step's second residual row: the projections that fold the norm in read one and write the other
    float *h = nullptr, *normed = nullptr, *P = nullptr, *qbuf = nullptr, *part = nullptr, *logits = nullptr, *emb_dev = nullptr;
    // A device-chained decode (GreedyChain* / SampleChain*): forwards queued ahead of the host, one token id coming back per forward
    struct Chain {
        static constexpr int DEPTH = 2; // forwards in flight: the one whose token is read next and one queued past it
        bool open = false, sample = false, in_call = false, exhausted = false;
        int slot = 0, next_pos = 0, exhausted_rc = 0;
        double temperature = 1;
        uint64_t seed = 0, draw_next = 0, draw_head = 0;
        unsigned head = 0, tail = 0; // forwards taken / queued
        int *host_ids = nullptr;     // pinned [DEPTH]
        hipEvent_t ev[DEPTH] = {};
    } chain;
    int kv_type = 0; // RD_KV_F16 or RD_KV_I8
    // Rows per step: up to ROWS_MAX as M-tiles of 32 (a dense model; MoE steps keep to one M-tile). The step's buffers hold
    // max_rows rows; partial sums and panels are per M-tile, pStride floats / xpStride bytes apart.
    static constexpr int ROWS_MAX = 512;
    int max_rows = 32;
    size_t pStride = 0, xpAStride = 0, xpBStride = 0;
    static constexpr int META_HDR = 3 * ROWS_MAX + ROWS_MAX * 6 + 8; // row slot, position, length, the rows' draw records (6 ints each), the expert bitmap
    int *rowDraw = nullptr;               // inside meta
    const rd_draw *step_draws = nullptr;  // set by the entry point for the one step it runs; null = plain argmax for every row
    void *XpA = nullptr, *XpB = nullptr;
    size_t P_floats = 0;
    float *cand_v = nullptr;
    int *cand_i = nullptr;
    int *ids = nullptr, *rowSlot = nullptr, *rowPos = nullptr, *rowLen = nullptr, *itemStart = nullptr;
    AttnItemH *items = nullptr;
    int *meta = nullptr; // one device block holding rowSlot, rowPos, rowLen, itemStart and items (one upload per step)
    size_t meta_ints = 0;
    int max_items = 0;
    // MoE scratch
    float *router_logits = nullptr, *moe_wgt = nullptr, *moe_gu = nullptr, *moe_dn = nullptr, *moe_out = nullptr;
    int *moe_idx = nullptr, *moe_idx_all = nullptr; // [32][k], [layers][32][k]
    signed char *moe_rank = nullptr;                 // [32][nE]
    bool last_logits_valid = false; // the last step wrote its rows' logits to `logits`
    int *topk_ids = nullptr;      // [max_rows][TOPK_MAX], the top-K of the last step's logits rows
    float *topk_vals = nullptr;
    double *topk_z = nullptr;
    TopkScratch topk_scratch;
    unsigned *moe_bits = nullptr;                    // inside meta: bitmap of the experts the current layer's routing chose (8 words)
    void *XpE = nullptr;                             // per-expert down panels
    float *XEf = nullptr;                            // per-row expert activations: [nE][32][expert_inter] f32 rows ahead of the per-row quantizer
    unsigned *moe_rowmax = nullptr;                  // [nE][32]: the bits of each such row's max |x| (cleared by the router's launch)
    // pinned host staging
    // STAGE_SLOTS slots used round-robin, so a caller that chains steps without reading anything back (the device greedy
    // chain) can enqueue several steps ahead of the GPU; a slot is rewritten only after its own upload has completed
    static constexpr int STAGE_SLOTS = 4;
    void *host_stage = nullptr;
    size_t host_stage_bytes = 0; // per slot
    size_t stage_meta_bytes = 0; // of which the metadata block (the embeddings follow)
    hipEvent_t stage_ev[STAGE_SLOTS] = {};
    bool stage_busy[STAGE_SLOTS] = {};
    unsigned stage_next = 0;
    int last_B = 0;

    // routing replay for the next step (rd_moe_replay): [layers] of host arrays the step uploads
    int replay_B = 0;
    std::vector<std::vector<int>> replay_idx;
    std::vector<std::vector<float>> replay_wgt;
    std::vector<std::vector<signed char>> replay_rank;

    StepTimer timer;
    // The step's attention work lists: [0] for the layers that read the whole context, [1] for the sliding-window layers (if any).
    // list_ints: ints between the two lists' (ranges, items) blocks in the metadata. The last step's lists stay on the device
    // (rd_bench_attn_chain replays them).
    size_t list_ints = 0, last_items[2] = {0, 0};
    bool last_grouped[2] = {false, false};
};
int launch_attn_partial(rd_model *m, const LayerW &l);

// multirow: a slot may carry several rows at consecutive positions (ragged verify / prefill rows)
int model_step(rd_model *m, int B, const int *slot, const int *pos, const float *emb_host, const float *emb_dev, int want, float *logits,
               int *ids, bool multirow = false);
