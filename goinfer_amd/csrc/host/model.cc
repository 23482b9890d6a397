// model.cc — the resident model: BuildResident's uploads (backend/cuda/backend.go:138-259), the paged KV pool
// (backend/cuda/kvpool.go) and the ragged batched decode step (backend/cuda/batchstep.go:49-78 StepBatch).
#include "model.h"
#include <algorithm>
#include <cmath>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define RC(x)                \
    do {                     \
        int rd_rc_macro_ = (x); \
        if (rd_rc_macro_) return rd_rc_macro_; \
    } while (0)

static int alloc_f32(rd_device *d, float **p, size_t n) { return d->alloc((void **)p, sizeof(float) * (n ? n : 1)); }

static bool graph_allowed() {
    if (getenv("ROCMDECODE_GRAPH")) return atoi(getenv("ROCMDECODE_GRAPH")) != 0;
    return !getenv("ROCP_TOOL_LIBRARIES");
}

extern "C" int rd_model_create(rd_device *d, const rd_model_desc *desc, rd_model **out) {
    if (!d || !desc || !out) return RD_ERR_ARG;
    const rd_model_desc &c = *desc;
    // Admission (goinfer's Admit gates, decoder/admit.go:36-48): what these kernels are built for.
    if (c.n_layers <= 0 || c.hidden <= 0 || c.hidden % 128 || c.hidden > 8192 || c.n_heads <= 0 || c.n_kv_heads <= 0 ||
        c.n_heads % c.n_kv_heads || (c.head_dim != 64 && c.head_dim != 128) || c.n_heads / c.n_kv_heads > 16 || c.vocab <= 0 || c.vocab % 32 ||
        !c.rope_inv_freq) {
        rd_set_error("rocm resident declines: needs hidden%%128==0 (<=8192), head_dim 64 or 128, GQA group <=16, vocab%%32==0");
        return RD_DECLINED;
    }
    if (c.n_experts > 0 && (c.n_experts > 256 || c.top_k <= 0 || c.top_k > c.n_experts || c.top_k > 64 || c.expert_inter % 128)) {
        rd_set_error("rocm resident declines: MoE needs <=256 experts and expert width %%128==0");
        return RD_DECLINED;
    }
    if (c.n_experts == 0 && (c.inter <= 0 || c.inter % 128)) {
        rd_set_error("rocm resident declines: FFN width must be a multiple of 128");
        return RD_DECLINED;
    }
    rd_model *m = new rd_model();
    m->d = d;
    // Graph replay is on unless the environment says otherwise, or a rocprofiler tool library is attached (ROCP_TOOL_LIBRARIES, as
    // rocprofv3 sets it): with kernel tracing on, replaying a captured graph ended in a segmentation fault inside the runtime on
    // ROCm 7.2, while the same program runs clean without the tool. ROCMDECODE_GRAPH=1 keeps it on regardless.
    m->graph.enabled = graph_allowed() && !getenv("ROCMDECODE_NO_GRAPH");
    m->desc = c;
    m->inv_freq.assign(c.rope_inv_freq, c.rope_inv_freq + c.head_dim / 2);
    m->desc.rope_inv_freq = nullptr;
    m->layers.resize((size_t)c.n_layers);
    for (auto &l : m->layers)
        if (c.n_experts > 0) l.exp_have.assign((size_t)c.n_experts * 3, 0);
    int rc = d->alloc((void **)&m->inv_freq_dev, sizeof(double) * m->inv_freq.size());
    if (!rc) rc = d->h2d(m->inv_freq_dev, m->inv_freq.data(), sizeof(double) * m->inv_freq.size());
    if (!rc) rc = d->alloc((void **)&m->rope_cs, sizeof(double) * 2 * (size_t)rd_model::ROWS_MAX * (c.head_dim / 2));
    if (!rc) rc = d->sync();
    if (rc) {
        delete m;
        return rc;
    }
    *out = m;
    return RD_OK;
}

extern "C" void rd_model_destroy(rd_model *m) {
    if (!m) return;
    rd_device *d = m->d;
    (void)d->sync();
    if (m->graph.exec) (void)d->hip->GraphExecDestroy(m->graph.exec);
    if (m->graph.graph) (void)d->hip->GraphDestroy(m->graph.graph);
    for (auto &l : m->layers) {
        free_weight(d, &l.qkv), free_weight(d, &l.o), free_weight(d, &l.gateup), free_weight(d, &l.down);
        for (void *p : {(void *)l.post_attn_norm, (void *)l.post_ffn_norm, (void *)l.attn_norm, (void *)l.ffn_norm, (void *)l.q_norm, (void *)l.k_norm, (void *)l.qkv_bias, (void *)l.router, (void *)l.router_bias, (void *)l.sinks, l.exp_gateup, l.exp_down,
                        (void *)l.Kp, (void *)l.Vp, (void *)l.Ksc, (void *)l.Vsc})
            d->release(p);
    }
    free_weight(d, &m->head);
    for (void *p : {(void *)m->embed_q, (void *)m->embed_scale, (void *)m->inv_freq_dev, (void *)m->rope_cs, (void *)m->final_norm, (void *)m->tables, (void *)m->h, (void *)m->h2, (void *)m->normed, (void *)m->P, (void *)m->qbuf,
                    (void *)m->part, (void *)m->attn_out, (void *)m->cand_v, (void *)m->cand_i, (void *)m->logits, (void *)m->emb_dev, m->XpA, m->XpB, (void *)m->ids, (void *)m->meta, (void *)m->router_logits, (void *)m->moe_wgt, (void *)m->moe_gu,
                    (void *)m->moe_dn, (void *)m->moe_out, (void *)m->moe_idx, (void *)m->moe_idx_all, (void *)m->moe_rank, (void *)m->topk_ids, (void *)m->topk_vals, (void *)m->topk_z, (void *)m->topk_scratch.ghist, (void *)m->topk_scratch.ccount, (void *)m->topk_scratch.gmax, (void *)m->topk_scratch.cand_i, (void *)m->topk_scratch.cand_v, (void *)m->topk_scratch.invT, (void *)m->topk_scratch.zpart, m->XpE, (void *)m->XEf, (void *)m->moe_rowmax})
        d->release(p);
    if (m->host_stage) (void)d->hip->HostFree(m->host_stage);
    if (m->chain.host_ids) (void)d->hip->HostFree(m->chain.host_ids);
    for (hipEvent_t e : m->chain.ev)
        if (e) (void)d->hip->EventDestroy(e);
    for (hipEvent_t e : m->stage_ev)
        if (e) (void)d->hip->EventDestroy(e);
    for (hipEvent_t e : m->timer.ev) (void)d->hip->EventDestroy(e);
    delete m;
}

// ---------------------------------------------------------------- uploads
static bool layer_ok(rd_model *m, int layer, bool allow_head) {
    if (allow_head && layer < 0) return true;
    if (layer < 0 || layer >= m->desc.n_layers) {
        rd_set_error("layer %d out of range", layer);
        return false;
    }
    return true;
}

static int expect_shape(rd_model *m, int proj, int N, int K) {
    const rd_model_desc &c = m->desc;
    int qd = c.n_heads * c.head_dim, kvd = c.n_kv_heads * c.head_dim;
    int wantN = 0, wantK = 0;
    switch (proj) {
    case RD_PROJ_Q: wantN = qd, wantK = c.hidden; break;
    case RD_PROJ_K:
    case RD_PROJ_V: wantN = kvd, wantK = c.hidden; break;
    case RD_PROJ_O: wantN = c.hidden, wantK = qd; break;
    case RD_PROJ_GATE:
    case RD_PROJ_UP: wantN = c.inter, wantK = c.hidden; break;
    case RD_PROJ_DOWN: wantN = c.hidden, wantK = c.inter; break;
    case RD_PROJ_HEAD: wantN = c.vocab, wantK = c.hidden; break;
    default: rd_set_error("unknown projection %d", proj); return RD_ERR_ARG;
    }
    if (N != wantN || K != wantK) {
        rd_set_error("projection %d: got %dx%d, model wants %dx%d", proj, N, K, wantN, wantK);
        return RD_ERR_ARG;
    }
    return RD_OK;
}

static int upload_pending(rd_device *d, const PendingMat &p, DevWeight *w) {
    if (p.kind == 0) return upload_q4k(d, p.data.data(), p.N, p.K, w);
    if (p.kind == 3) return upload_q5k(d, p.data.data(), p.N, p.K, w);
    if (p.kind == 4) return upload_q6k(d, p.data.data(), p.N, p.K, w);
    if (p.kind == 1) return upload_w8a8(d, (const int8_t *)p.data.data(), (const float *)p.scales.data(), p.N, p.K, w, p.act_group);
    return upload_w4a8(d, p.data.data(), (const uint16_t *)p.scales.data(), p.N, p.K, w, false, p.act_group);
}

// Concatenate row-wise (all kinds are row-major with per-row side data) and upload as one weight. Members of different
// kinds (a GGUF Q4_K_M file stores some attn_v as Q6_K, and goinfer's q4k mode turns those into int8 copies) become a group:
// each run of one kind is its own weight, multiplied by its own kernel into the group's shared partial-sum buffer.
static int fuse_and_upload(rd_device *d, PendingMat *parts, int n, DevWeight *w) {
    auto group_of = [](const PendingMat &p) { return p.kind == 1 || p.kind == 2 ? p.act_group : 32; }; // K-quants are per-32 by kind
    for (int i = 1; i < n; i++) {
        if (parts[i].K != parts[0].K) {
            rd_set_error("rocm resident declines: fused projections differ in K");
            return RD_DECLINED;
        }
        if (group_of(parts[i]) != group_of(parts[0])) { // one quantizer feeds them all
            rd_set_error("rocm resident declines: fused projections differ in activation quantization group (%d and %d)", group_of(parts[0]), group_of(parts[i]));
            return RD_DECLINED;
        }
    }
    std::vector<PendingMat> runs;
    for (int i = 0; i < n; i++) {
        if (runs.empty() || runs.back().kind != parts[i].kind) {
            runs.emplace_back();
            runs.back().kind = parts[i].kind, runs.back().K = parts[i].K, runs.back().N = 0, runs.back().act_group = parts[i].act_group;
        }
        PendingMat &cat = runs.back();
        cat.N += parts[i].N;
        cat.data.insert(cat.data.end(), parts[i].data.begin(), parts[i].data.end());
        cat.scales.insert(cat.scales.end(), parts[i].scales.begin(), parts[i].scales.end());
    }
    int rc = RD_OK;
    if (runs.size() == 1) {
        rc = upload_pending(d, runs[0], w);
    } else {
        DevWeight g;
        g.kind = WKIND_GROUP, g.K = parts[0].K, g.N = 0;
        for (auto &r : runs) {
            g.parts.emplace_back();
            g.col0.push_back(g.N);
            if ((rc = upload_pending(d, r, &g.parts.back()))) break;
            g.N += r.N;
        }
        if (rc)
            free_weight(d, &g);
        else
            *w = std::move(g);
    }
    if (!rc)
        for (int i = 0; i < n; i++) parts[i] = PendingMat(), parts[i].kind = -2; // consumed
    return rc;
}

// The rows of a q, k or v projection reordered within each head so that a rotation pair (d, d + hd/2) lands in one 32-row GEMM
// tile, sixteen rows apart: new row 32j + l of a head holds d = 16j + l for l < 16 and d = hd/2 + 16j + (l - 16) above
// (qkv_col in the kernels is the inverse). The fused q|k|v kernel rotates the pair inside the tile that produced it.
static void permute_head_rows(PendingMat *p, int hd) {
    const size_t rowB = p->data.size() / (size_t)p->N, scB = p->scales.size() / (size_t)p->N;
    std::vector<uint8_t> data(p->data.size()), scales(p->scales.size());
    const int half = hd / 2;
    for (int n = 0; n < p->N; n++) {
        const int head = n / hd, c = n % hd, j = c >> 5, l = c & 31;
        const int src = head * hd + (l < 16 ? 16 * j + l : half + 16 * j + (l - 16));
        memcpy(&data[(size_t)n * rowB], &p->data[(size_t)src * rowB], rowB);
        if (scB) memcpy(&scales[(size_t)n * scB], &p->scales[(size_t)src * scB], scB);
    }
    p->data.swap(data), p->scales.swap(scales);
}

static int accept(rd_model *m, int layer, int proj, PendingMat &&pm) {
    if (m->finalized) {
        rd_set_error("model already finalized");
        return RD_ERR_STATE;
    }
    rd_device *d = m->d;
    if (proj == RD_PROJ_HEAD) {
        free_weight(d, &m->head);
        return upload_pending(d, pm, &m->head);
    }
    LayerW &l = m->layers[(size_t)layer];
    if (proj == RD_PROJ_O) {
        free_weight(d, &l.o);
        return upload_pending(d, pm, &l.o);
    }
    if (proj == RD_PROJ_DOWN) {
        free_weight(d, &l.down);
        return upload_pending(d, pm, &l.down);
    }
    l.pend[proj] = std::move(pm);
    if (proj <= RD_PROJ_V) {
        permute_head_rows(&l.pend[proj], m->desc.head_dim);
        if (l.pend[RD_PROJ_Q].kind >= 0 && l.pend[RD_PROJ_K].kind >= 0 && l.pend[RD_PROJ_V].kind >= 0) {
            free_weight(d, &l.qkv);
            return fuse_and_upload(d, &l.pend[RD_PROJ_Q], 3, &l.qkv);
        }
    } else if (l.pend[RD_PROJ_GATE].kind >= 0 && l.pend[RD_PROJ_UP].kind >= 0) {
        free_weight(d, &l.gateup);
        return fuse_and_upload(d, &l.pend[RD_PROJ_GATE], 2, &l.gateup);
    }
    return RD_OK;
}

extern "C" int rd_model_upload_q4k(rd_model *m, int layer, int proj, const void *blocks, int N, int K) {
    if (!m || !blocks) return RD_ERR_ARG;
    if (!layer_ok(m, layer, proj == RD_PROJ_HEAD)) return RD_ERR_ARG;
    RC(expect_shape(m, proj, N, K));
    if (K % 256) {
        rd_set_error("Q4_K needs K%%256==0 (goinfer kquant_native.go:88-90), got K=%d", K);
        return RD_DECLINED;
    }
    PendingMat pm;
    pm.kind = 0, pm.N = N, pm.K = K;
    pm.data.assign((const uint8_t *)blocks, (const uint8_t *)blocks + (size_t)N * (K / 256) * 144);
    return accept(m, layer, proj, std::move(pm));
}

static int upload_kquant(rd_model *m, int layer, int proj, const void *blocks, int N, int K, int kind, int bb, const char *name) {
    if (!m || !blocks) return RD_ERR_ARG;
    if (!layer_ok(m, layer, proj == RD_PROJ_HEAD)) return RD_ERR_ARG;
    RC(expect_shape(m, proj, N, K));
    if (K % 256) {
        rd_set_error("%s needs K%%256==0 (goinfer kquant_native.go:88-90), got K=%d", name, K);
        return RD_DECLINED;
    }
    PendingMat pm;
    pm.kind = kind, pm.N = N, pm.K = K;
    pm.data.assign((const uint8_t *)blocks, (const uint8_t *)blocks + (size_t)N * (K / 256) * bb);
    return accept(m, layer, proj, std::move(pm));
}
extern "C" int rd_model_upload_q5k(rd_model *m, int layer, int proj, const void *blocks, int N, int K) {
    return upload_kquant(m, layer, proj, blocks, N, K, 3, 176, "Q5_K");
}
extern "C" int rd_model_upload_q6k(rd_model *m, int layer, int proj, const void *blocks, int N, int K) {
    return upload_kquant(m, layer, proj, blocks, N, K, 4, 210, "Q6_K");
}

extern "C" int rd_model_upload_w8a8(rd_model *m, int layer, int proj, const int8_t *q, const float *row_scale, int N, int K) {
    if (!m || !q || !row_scale) return RD_ERR_ARG;
    if (!layer_ok(m, layer, proj == RD_PROJ_HEAD)) return RD_ERR_ARG;
    RC(expect_shape(m, proj, N, K));
    PendingMat pm;
    pm.kind = 1, pm.N = N, pm.K = K, pm.act_group = m->upload_act_group;
    pm.data.assign((const uint8_t *)q, (const uint8_t *)q + (size_t)N * K);
    pm.scales.assign((const uint8_t *)row_scale, (const uint8_t *)row_scale + sizeof(float) * (size_t)N);
    return accept(m, layer, proj, std::move(pm));
}

extern "C" int rd_model_upload_w4a8(rd_model *m, int layer, int proj, int expert, const uint8_t *nib, const uint16_t *s16, int N, int K) {
    if (!m || !nib || !s16) return RD_ERR_ARG;
    if (!layer_ok(m, layer, proj == RD_PROJ_HEAD && expert < 0)) return RD_ERR_ARG;
    rd_device *d = m->d;
    const rd_model_desc &c = m->desc;
    if (expert < 0) {
        RC(expect_shape(m, proj, N, K));
        PendingMat pm;
        pm.kind = 2, pm.N = N, pm.K = K, pm.act_group = m->upload_act_group;
        pm.data.assign(nib, nib + (size_t)N * K / 2);
        pm.scales.assign((const uint8_t *)s16, (const uint8_t *)s16 + 2 * (size_t)N * (K / 32));
        return accept(m, layer, proj, std::move(pm));
    }
    // expert tensors: gate and up are stacked [gate; up] per expert (one GEMM), down is its own stack
    if (c.n_experts <= 0 || expert >= c.n_experts || (proj != RD_PROJ_GATE && proj != RD_PROJ_UP && proj != RD_PROJ_DOWN)) {
        rd_set_error("bad expert upload (expert %d, proj %d)", expert, proj);
        return RD_ERR_ARG;
    }
    int I = c.expert_inter, H = c.hidden;
    bool isDown = proj == RD_PROJ_DOWN;
    if ((isDown && (N != H || K != I)) || (!isDown && (N != I || K != H))) {
        rd_set_error("expert projection %d: got %dx%d", proj, N, K);
        return RD_ERR_ARG;
    }
    if (m->exp_act_group >= 0 && m->exp_act_group != m->upload_act_group) {
        rd_set_error("rocm resident declines: expert tensors differ in activation quantization group (%d and %d)", m->exp_act_group, m->upload_act_group);
        return RD_DECLINED;
    }
    if (m->upload_act_group == 0 && I > 8192) {
        rd_set_error("rocm resident declines: per-row expert activations with expert width %d (at most 8192)", I);
        return RD_DECLINED;
    }
    m->exp_act_group = m->upload_act_group;
    LayerW &l = m->layers[(size_t)layer];
    size_t guBytes = (size_t)(2 * I / 32) * ((H + 255) / 256) * 4608, dnBytes = (size_t)(H / 32) * ((I + 255) / 256) * 4608;
    if (!l.exp_gateup) {
        RC(d->alloc(&l.exp_gateup, guBytes * c.n_experts));
        RC(d->alloc(&l.exp_down, dnBytes * c.n_experts));
    }
    if (K > MOE_GEMV_MAX_K) {
        rd_set_error("rocm resident declines: expert projection with K=%d (at most %d)", K, MOE_GEMV_MAX_K);
        return RD_DECLINED;
    }
    DevWeight tmp;
    RC(upload_w4a8(d, nib, s16, N, K, &tmp, true));
    size_t tb = (size_t)(N / 32) * ((K + 255) / 256) * 4608;
    uint8_t *dst = isDown ? (uint8_t *)l.exp_down + dnBytes * expert
                          : (uint8_t *)l.exp_gateup + guBytes * expert + (proj == RD_PROJ_UP ? guBytes / 2 : 0);
    int rc = rd_hip_ok(d->hip, d->hip->MemcpyAsync(dst, tmp.tiled, tb, hipMemcpyDeviceToDevice, d->stream), "expert copy") ? RD_OK : RD_ERR_HIP;
    if (!rc) rc = d->sync();
    free_weight(d, &tmp);
    if (!rc) l.exp_have[(size_t)expert * 3 + (proj == RD_PROJ_GATE ? 0 : proj == RD_PROJ_UP ? 1 : 2)] = 1;
    return rc;
}

extern "C" int rd_model_upload_f32(rd_model *m, int layer, int which, const float *v, size_t n) {
    if (!m || !v) return RD_ERR_ARG;
    rd_device *d = m->d;
    const rd_model_desc &c = m->desc;
    float **slot = nullptr;
    size_t want = 0;
    if (which == RD_VEC_FINAL_NORM) {
        slot = &m->final_norm, want = (size_t)c.hidden;
    } else {
        if (!layer_ok(m, layer, false)) return RD_ERR_ARG;
        LayerW &l = m->layers[(size_t)layer];
        switch (which) {
        case RD_VEC_ATTN_NORM: slot = &l.attn_norm, want = (size_t)c.hidden; break;
        case RD_VEC_FFN_NORM: slot = &l.ffn_norm, want = (size_t)c.hidden; break;
        case RD_VEC_Q_NORM: slot = &l.q_norm, want = (size_t)c.head_dim; break;
        case RD_VEC_K_NORM: slot = &l.k_norm, want = (size_t)c.head_dim; break;
        case RD_VEC_QKV_BIAS: slot = &l.qkv_bias, want = (size_t)(c.n_heads + 2 * c.n_kv_heads) * c.head_dim; break;
        case RD_VEC_ROUTER: slot = &l.router, want = (size_t)c.n_experts * c.hidden; break;
        case RD_VEC_ROUTER_BIAS: slot = &l.router_bias, want = (size_t)c.n_experts; break;
        case RD_VEC_ATTN_SINKS: slot = &l.sinks, want = (size_t)c.n_heads; break;
        case RD_VEC_POST_ATTN_NORM: slot = &l.post_attn_norm, want = (size_t)c.hidden; break;
        case RD_VEC_POST_FFN_NORM: slot = &l.post_ffn_norm, want = (size_t)c.hidden; break;
        default: rd_set_error("unknown vector %d", which); return RD_ERR_ARG;
        }
    }
    if (n != want) {
        rd_set_error("vector %d: got %zu values, want %zu", which, n, want);
        return RD_ERR_ARG;
    }
    if (m->finalized) { // the (1 + w) pass has run over the norm weights: a later upload would skip it
        rd_set_error("model already finalized");
        return RD_ERR_STATE;
    }
    if (!*slot) RC(alloc_f32(d, slot, n));
    RC(d->h2d(*slot, v, sizeof(float) * n));
    return d->sync();
}

// WeightMat.ActQuantGroup() of the int8 / int4 tensors uploaded from here on (decoder/weightmat.go:837,909,936): 32 = activations
// quantized per group of 32 (goinfer's q4k mode), 0 = one scale per row (its int8 / int4 modes, and the lane its staged
// QuantBackend / QuantBackend4 hooks serve: decoder/backend.go:38-88).
extern "C" int rd_model_set_act_group(rd_model *m, int act_group) {
    if (!m) return RD_ERR_ARG;
    if (m->finalized) {
        rd_set_error("model already finalized");
        return RD_ERR_STATE;
    }
    if (act_group != 0 && act_group != 32) {
        rd_set_error("rocm resident declines: activation quantization group %d (32 = per group of 32, 0 = one scale per row)", act_group);
        return RD_DECLINED;
    }
    m->upload_act_group = act_group;
    return RD_OK;
}

// The router's variant (decoder/mlp.go:130-228 routeExperts / groupLimit), before rd_model_finalize.
extern "C" int rd_model_set_router(rd_model *m, int sigmoid, double scale, int n_group, int topk_group) {
    if (!m) return RD_ERR_ARG;
    if (m->finalized) {
        rd_set_error("model already finalized");
        return RD_ERR_STATE;
    }
    if (n_group > 32 || (n_group > 1 && (topk_group < 1 || topk_group > n_group || m->desc.n_experts % n_group))) {
        rd_set_error("rocm resident declines: group-limited routing takes 2..32 groups that divide the experts, and 1..n_group of them");
        return RD_DECLINED;
    }
    m->router_sigmoid = sigmoid ? 1 : 0, m->router_scale = (float)scale, m->n_group = n_group > 1 ? n_group : 0, m->topk_group = topk_group;
    return RD_OK;
}

// The block's family knobs (Gemma; backend/cuda/resident.go:549-565 finalSoftcap, act, addOneArg), before rd_model_finalize.
extern "C" int rd_model_set_block(rd_model *m, int norm_add_one, int act, float final_softcap, double logit_scale) {
    if (!m || (act != RD_ACT_SILU && act != RD_ACT_GELU_TANH) || !(final_softcap >= 0.f) || !(logit_scale >= 0.0)) return RD_ERR_ARG;
    if (m->finalized) {
        rd_set_error("model already finalized");
        return RD_ERR_STATE;
    }
    if (act != RD_ACT_SILU && m->desc.n_experts > 0) {
        rd_set_error("rocm resident declines: a GeGLU mixture-of-experts block");
        return RD_DECLINED;
    }
    m->norm_add_one = norm_add_one ? 1 : 0, m->act = act, m->final_softcap = final_softcap;
    m->logit_mul = (logit_scale != 0.0 && logit_scale != 1.0) ? (float)(1 / logit_scale) : 0.f;
    return RD_OK;
}

// A sliding-window layer (kvmgr.WindowNeedStart, internal/runtime/kvmgr/sequence.go:55-60): the layer's rows read the last
// `window` positions only. Before rd_model_finalize; the windowed layers of a model share one window length.
extern "C" int rd_model_set_window(rd_model *m, int layer, int window) {
    if (!m || !layer_ok(m, layer, false) || window < 0) return RD_ERR_ARG;
    if (m->finalized) {
        rd_set_error("model already finalized");
        return RD_ERR_STATE;
    }
    // the model's window is what its layers hold now: a layer set back to 0 no longer counts
    m->layers[(size_t)layer].window = 0;
    m->window = 0;
    for (const LayerW &l : m->layers) m->window = std::max(m->window, l.window);
    if (window > 0 && m->window > 0 && window != m->window) {
        rd_set_error("rocm resident declines: sliding-window layers of different lengths (%d and %d)", m->window, window);
        return RD_DECLINED;
    }
    m->layers[(size_t)layer].window = window;
    m->window = std::max(m->window, window);
    return RD_OK;
}

// The int8 embedding table, resident so a greedy chain can run without the host (goinfer's GreedyChain*,
// decoder/resident/subsystems.go:78-100); the ordinary step still takes host embedding rows.
extern "C" int rd_model_upload_embedding(rd_model *m, const int8_t *q, const float *row_scale) {
    if (!m || !q || !row_scale) return RD_ERR_ARG;
    rd_device *d = m->d;
    size_t V = (size_t)m->desc.vocab, H = (size_t)m->desc.hidden;
    if (!m->embed_q) {
        RC(d->alloc((void **)&m->embed_q, V * H));
        RC(d->alloc((void **)&m->embed_scale, sizeof(float) * V));
    }
    RC(d->h2d(m->embed_q, q, V * H));
    RC(d->h2d(m->embed_scale, row_scale, sizeof(float) * V));
    return d->sync();
}

// A group's members all run with one split count, so that the consumer sums the same number of partials for every column: the
// fewest any member's own plan asks for (no member then gets more splits than it has K-blocks).
static GemmPlan group_plan(const DevWeight &w) {
    GemmPlan g{1 << 30, 0, 0};
    for (const auto &p : w.parts) g.splits = std::min(g.splits, plan_gemm(p.kind, p.N, kblocks_for(p), p.act_group).splits);
    return g;
}

static size_t gemm_partial_floats(const DevWeight &w) {
    if (w.kind < 0) return 0;
    if (w.kind == WKIND_GROUP) return (size_t)group_plan(w).splits * 32 * w.N;
    int nKB = kblocks_for(w);
    return (size_t)plan_gemm(w.kind, w.N, nKB, w.act_group).splits * 32 * w.N;
}

extern "C" int rd_model_finalize(rd_model *m) {
    if (!m) return RD_ERR_ARG;
    rd_device *d = m->d;
    const rd_model_desc &c = m->desc;
    size_t pf = 0;
    for (int i = 0; i < c.n_layers; i++) {
        LayerW &l = m->layers[(size_t)i];
        bool ok = l.qkv.kind >= 0 && l.o.kind >= 0 && l.attn_norm && l.ffn_norm && (!c.qk_norm || (l.q_norm && l.k_norm));
        if (c.n_experts == 0)
            ok = ok && l.gateup.kind >= 0 && l.down.kind >= 0;
        else {
            ok = ok && l.router && l.exp_gateup;
            for (char hv : l.exp_have) ok = ok && hv;
        }
        if (!ok) {
            rd_set_error("layer %d is missing tensors", i);
            return RD_ERR_STATE;
        }
        if (c.n_experts > 0 && (l.post_attn_norm || l.post_ffn_norm)) {
            rd_set_error("rocm resident declines: post-branch norms around a mixture-of-experts block");
            return RD_DECLINED;
        }
        pf = std::max({pf, gemm_partial_floats(l.qkv), gemm_partial_floats(l.o), gemm_partial_floats(l.gateup), gemm_partial_floats(l.down)});
    }
    if (m->head.kind < 0 || !m->final_norm) {
        rd_set_error("model is missing the head or the final norm");
        return RD_ERR_STATE;
    }
    pf = std::max(pf, gemm_partial_floats(m->head));
    int H = c.hidden, qd = c.n_heads * c.head_dim;
    m->max_rows = c.n_experts > 0 ? 32 : rd_model::ROWS_MAX;
    const size_t R = (size_t)m->max_rows, tiles = R / 32;
    m->P_floats = pf;
    m->pStride = pf;
    RC(alloc_f32(d, &m->P, pf * tiles));
    RC(alloc_f32(d, &m->h, R * H));
    RC(alloc_f32(d, &m->h2, (size_t)H));
    RC(alloc_f32(d, &m->emb_dev, R * H));
    RC(alloc_f32(d, &m->normed, (size_t)32 * H));
    RC(alloc_f32(d, &m->qbuf, R * qd));
    if (std::any_of(m->layers.begin(), m->layers.end(), [](const LayerW &l) { return act_group_for(l.o) == 0; })) RC(alloc_f32(d, &m->attn_out, R * qd));
    RC(alloc_f32(d, &m->logits, R * c.vocab));
    size_t kA = (size_t)H, kB = (size_t)std::max(qd, c.n_experts ? qd : c.inter);
    auto panel_room = [](size_t K) { return a8_bytes((int)K); };
    m->xpAStride = panel_room(kA), m->xpBStride = panel_room(kB);
    RC(d->alloc(&m->XpA, m->xpAStride * tiles));
    RC(d->alloc(&m->XpB, m->xpBStride * tiles));
    // An A8 panel's last block is written only up to K: what lies past it (K not a multiple of 256) must hold finite scales and
    // sums for good, since the GEMM multiplies them with the weights' zero padding.
    HIPCHK(MemsetAsync(m->XpA, 0, m->xpAStride * tiles, d->stream));
    HIPCHK(MemsetAsync(m->XpB, 0, m->xpBStride * tiles, d->stream));
    RC(d->alloc((void **)&m->ids, sizeof(int) * R));
    RC(alloc_f32(d, &m->cand_v, R * ((c.vocab + 4095) / 4096)));
    RC(d->alloc((void **)&m->cand_i, sizeof(int) * R * (size_t)((c.vocab + 4095) / 4096)));
    if (c.n_experts > 0) {
        int k = c.top_k, I = c.expert_inter;
        RC(alloc_f32(d, &m->router_logits, (size_t)32 * c.n_experts));
        RC(alloc_f32(d, &m->moe_wgt, (size_t)32 * k));
        RC(alloc_f32(d, &m->moe_gu, (size_t)32 * k * 2 * I));
        RC(alloc_f32(d, &m->moe_dn, (size_t)32 * k * H));
        RC(alloc_f32(d, &m->moe_out, (size_t)32 * H));
        RC(d->alloc((void **)&m->moe_idx, sizeof(int) * 32 * k));
        RC(d->alloc((void **)&m->moe_idx_all, sizeof(int) * (size_t)c.n_layers * 32 * k));
        RC(d->alloc((void **)&m->moe_rank, (size_t)32 * c.n_experts));
        RC(d->alloc(&m->XpE, (size_t)c.n_experts * a8_bytes(I)));
        HIPCHK(MemsetAsync(m->XpE, 0, (size_t)c.n_experts * a8_bytes(I), d->stream));
        if (m->exp_act_group == 0) {
            RC(alloc_f32(d, &m->XEf, (size_t)c.n_experts * 32 * I));
            RC(d->alloc((void **)&m->moe_rowmax, sizeof(unsigned) * (size_t)c.n_experts * 32));
            HIPCHK(MemsetAsync(m->moe_rowmax, 0, sizeof(unsigned) * (size_t)c.n_experts * 32, d->stream));
        }
    }
    RC(d->alloc((void **)&m->topk_ids, sizeof(int) * R * TOPK_MAX));
    RC(alloc_f32(d, &m->topk_vals, R * TOPK_MAX));
    RC(topk_scratch_alloc(d, (int)R, c.vocab, &m->topk_scratch));
    RC(d->alloc((void **)&m->topk_z, sizeof(double) * R));
    for (auto &e : m->stage_ev) HIPCHK(EventCreate(&e));
    if (m->norm_add_one && !m->ones_added) {
        // Gemma stores every RMSNorm weight as its deviation from one; the norm scales by f32(1 + w) (decoder/rmsnorm.go:62-75),
        // so the sum is formed once here and the kernels multiply by it as they do by a plain weight
        auto bump = [&](float *w, int n) -> int {
            return w ? d->launch(d->k.add_one, (unsigned)((n + 255) / 256), 1, 1, 256, w, n) : RD_OK;
        };
        for (LayerW &l : m->layers) {
            for (float *w : {l.attn_norm, l.ffn_norm, l.post_attn_norm, l.post_ffn_norm}) RC(bump(w, H));
            RC(bump(l.q_norm, c.head_dim));
            RC(bump(l.k_norm, c.head_dim));
        }
        RC(bump(m->final_norm, H));
        m->ones_added = true;
    }
    m->finalized = true;
    return d->sync();
}

// ---------------------------------------------------------------- KV
extern "C" int rd_kv_configure(rd_model *m, int slots, int ctx_cap) { return rd_kv_configure_typed(m, slots, ctx_cap, RD_KV_F16); }

extern "C" int rd_kv_configure_typed(rd_model *m, int slots, int ctx_cap, int kv_type) {
    if (!m || slots <= 0 || ctx_cap <= 0) return RD_ERR_ARG;
    if (kv_type != RD_KV_F16 && kv_type != RD_KV_I8) {
        rd_set_error("rd_kv_configure_typed: unknown KV type %d", kv_type);
        return RD_ERR_ARG;
    }
    if (m->tables) {
        rd_set_error("KV already configured");
        return RD_ERR_STATE;
    }
    // The work list, the partial-sum area, the metadata block and the pinned staging slots are sized from the widest step the
    // model takes, which rd_model_finalize settles: configuring first would size them for a narrower step than the model runs.
    if (!m->finalized) {
        rd_set_error("rd_kv_configure before rd_model_finalize");
        return RD_ERR_STATE;
    }
    rd_device *d = m->d;
    RC(d->use());
    const rd_model_desc &c = m->desc;
    m->slots = slots, m->ctx_cap = ctx_cap, m->blocks_per_slot = (ctx_cap + 63) / 64;
    size_t nBlocks = (size_t)slots * m->blocks_per_slot + 1; // block 0 is the all-zero block no slot owns
    const bool i8 = kv_type == RD_KV_I8;
    size_t bytes = nBlocks * c.n_kv_heads * 64 * c.head_dim * (i8 ? 1 : 2);
    size_t scBytes = i8 ? nBlocks * c.n_kv_heads * 64 * sizeof(float) : 0;
    m->kv_type = kv_type;
    size_t fr = 0, tot = 0;
    HIPCHK(MemGetInfo(&fr, &tot));
    if ((bytes + scBytes) * 2 * c.n_layers > fr) {
        rd_set_error("rocm resident declines: KV pool of %zu MiB exceeds free device memory (%zu MiB)", ((bytes + scBytes) * 2 * c.n_layers) >> 20, fr >> 20);
        return RD_DECLINED;
    }
    for (auto &l : m->layers) {
        RC(d->alloc((void **)&l.Kp, bytes));
        RC(d->alloc((void **)&l.Vp, bytes));
        HIPCHK(MemsetAsync(l.Kp, 0, bytes, d->stream));
        HIPCHK(MemsetAsync(l.Vp, 0, bytes, d->stream));
        if (i8) {
            RC(d->alloc((void **)&l.Ksc, scBytes));
            RC(d->alloc((void **)&l.Vsc, scBytes));
            HIPCHK(MemsetAsync(l.Ksc, 0, scBytes, d->stream));
            HIPCHK(MemsetAsync(l.Vsc, 0, scBytes, d->stream));
        }
    }
    // Static ownership: slot s owns blocks 1+s*bps .. ; the table indirection stays so a pool allocator can replace it.
    std::vector<int> tab((size_t)slots * m->blocks_per_slot);
    for (size_t i = 0; i < tab.size(); i++) tab[i] = (int)(i + 1);
    RC(d->alloc((void **)&m->tables, sizeof(int) * tab.size()));
    RC(d->h2d(m->tables, tab.data(), sizeof(int) * tab.size()));
    m->slot_len.assign((size_t)slots, 0);
    // attention work list: every (row, kv head) of a step is cut into at most attn_max_pieces items
    m->max_items = m->max_rows * c.n_kv_heads * attn_max_pieces(m->blocks_per_slot);
    m->max_items = (m->max_items + ATTN_LIST_PAD - 1) / ATTN_LIST_PAD * ATTN_LIST_PAD; // a step's list is padded to this grain
    RC(alloc_f32(d, &m->part, (size_t)m->max_items * ATTN_TILE_ROWS * (c.head_dim + 2)));
    // The step's metadata lives in one device block so a step uploads it with one copy:
    // [row slot R][row position R][row length R][row draw records R x 6][item ranges max_rows*nKV*3][items max_items x 4] ints, R = ROWS_MAX
    const size_t rangeInts = (size_t)m->max_rows * c.n_kv_heads * ATTN_RANGE_INTS;
    m->list_ints = rangeInts + (size_t)m->max_items * 4;
    m->meta_ints = rd_model::META_HDR + m->list_ints * (m->window > 0 ? 2 : 1); // a second work list for the sliding-window layers
    RC(d->alloc((void **)&m->meta, sizeof(int) * m->meta_ints));
    constexpr int RM = rd_model::ROWS_MAX;
    m->rowSlot = m->meta, m->rowPos = m->meta + RM, m->rowLen = m->meta + 2 * RM, m->rowDraw = m->meta + 3 * RM;
    m->moe_bits = (unsigned *)(m->meta + rd_model::META_HDR - 8);
    m->itemStart = m->meta + rd_model::META_HDR;
    m->items = (AttnItemH *)(m->meta + rd_model::META_HDR + rangeInts);
    // pinned staging, STAGE_SLOTS slots: the step's metadata block as on the device, then the embeddings
    m->stage_meta_bytes = (sizeof(int) * m->meta_ints + 4095) & ~(size_t)4095;
    m->host_stage_bytes = m->stage_meta_bytes + sizeof(float) * (size_t)m->max_rows * c.hidden;
    HIPCHK(HostMalloc(&m->host_stage, m->host_stage_bytes * rd_model::STAGE_SLOTS, 0));
    return d->sync();
}

static bool slot_ok(rd_model *m, int slot) {
    if (!m->tables || slot < 0 || slot >= m->slots) {
        rd_set_error("KV slot %d out of range (configured %d)", slot, m->slots);
        return false;
    }
    return true;
}

extern "C" int rd_kv_upload(rd_model *m, int slot, int layer, int base, int n, const float *keys, const float *vals) {
    if (!m || !keys || !vals || n <= 0 || base < 0) return RD_ERR_ARG;
    if (!slot_ok(m, slot) || !layer_ok(m, layer, false)) return RD_ERR_ARG;
    if (base + n > m->ctx_cap) {
        rd_set_error("rd_kv_upload: positions %d..%d exceed the context cap %d", base, base + n - 1, m->ctx_cap);
        return RD_ERR_KV_FULL;
    }
    rd_device *d = m->d;
    const rd_model_desc &c = m->desc;
    int kvd = c.n_kv_heads * c.head_dim;
    DevBuf K(d), V(d);
    RC(K.alloc(sizeof(float) * (size_t)n * kvd));
    RC(V.alloc(sizeof(float) * (size_t)n * kvd));
    RC(d->h2d(K.p, keys, sizeof(float) * (size_t)n * kvd));
    RC(d->h2d(V.p, vals, sizeof(float) * (size_t)n * kvd));
    LayerW &l = m->layers[(size_t)layer];
    if (m->kv_type == RD_KV_I8)
        RC(d->launch(d->k.kv_store_i8, (unsigned)n, (unsigned)c.n_kv_heads, 1, 64, (const float *)K.p, (const float *)V.p, (signed char *)l.Kp,
                     (signed char *)l.Vp, l.Ksc, l.Vsc, (const int *)(m->tables + (size_t)slot * m->blocks_per_slot), base, c.n_kv_heads, c.head_dim));
    else
        RC(d->launch(d->k.kv_store, (unsigned)n, (unsigned)c.n_kv_heads, 1, (unsigned)c.head_dim, (const float *)K.p, (const float *)V.p, l.Kp, l.Vp,
                     (const int *)(m->tables + (size_t)slot * m->blocks_per_slot), base, c.n_kv_heads, c.head_dim));
    RC(d->sync());
    m->slot_len[(size_t)slot] = std::max(m->slot_len[(size_t)slot], base + n);
    return RD_OK;
}

// The host copy of rows a slot holds (decoder/resident/subsystems.go:280-287 SnapshotKV takes one per layer): what the cache
// stores, widened to f32 the way an attention read sees it.
extern "C" int rd_kv_download(rd_model *m, int slot, int layer, int base, int n, float *keys, float *vals) {
    if (!m || !keys || !vals || n <= 0 || base < 0) return RD_ERR_ARG;
    if (!slot_ok(m, slot) || !layer_ok(m, layer, false)) return RD_ERR_ARG;
    if (base + n > m->slot_len[(size_t)slot]) {
        rd_set_error("rd_kv_download: rows %d..%d, slot %d holds %d", base, base + n - 1, slot, m->slot_len[(size_t)slot]);
        return RD_ERR_ARG;
    }
    rd_device *d = m->d;
    RC(d->use());
    const rd_model_desc &c = m->desc;
    const size_t bytes = sizeof(float) * (size_t)n * c.n_kv_heads * c.head_dim;
    DevBuf K(d), V(d);
    RC(K.alloc(bytes));
    RC(V.alloc(bytes));
    LayerW &l = m->layers[(size_t)layer];
    RC(d->launch(d->k.kv_read, (unsigned)n, (unsigned)c.n_kv_heads, 1, (unsigned)c.head_dim, (const void *)l.Kp, (const void *)l.Vp, (const float *)l.Ksc,
                 (const float *)l.Vsc, K.as<float>(), V.as<float>(), (const int *)(m->tables + (size_t)slot * m->blocks_per_slot), base, c.n_kv_heads,
                 c.head_dim, m->kv_type == RD_KV_I8 ? 1 : 0));
    RC(d->d2h(keys, K.p, bytes));
    return d->d2h(vals, V.p, bytes);
}

extern "C" int rd_kv_truncate(rd_model *m, int slot, int pos) {
    if (!m || !slot_ok(m, slot) || pos < 0) return RD_ERR_ARG;
    m->slot_len[(size_t)slot] = std::min(m->slot_len[(size_t)slot], pos);
    return RD_OK;
}

extern "C" int rd_kv_reset(rd_model *m, int slot) { return rd_kv_truncate(m, slot, 0); }

// ---------------------------------------------------------------- the step
struct Scope { // times one kernel class when the model's timer is on
    rd_model *m;
    int cls;
    Scope(rd_model *mm, int c) : m(mm), cls(c) {
        if (!m->timer.on) return;
        hipEvent_t a, b;
        (void)m->d->hip->EventCreate(&a), (void)m->d->hip->EventCreate(&b);
        m->timer.ev.push_back(a), m->timer.ev.push_back(b), m->timer.cls.push_back(cls);
        (void)m->d->hip->EventRecord(a, m->d->stream);
    }
    ~Scope() {
        if (m->timer.on) (void)m->d->hip->EventRecord(m->timer.ev.back(), m->d->stream);
    }
};

// *grouped: some item covers several positions of one sequence (the step then runs the attention kernels for such items).
static int build_attn_items(rd_model *m, int B, const int *slot, const int *pos, std::vector<AttnItemH> &items, std::vector<int> &ranges, bool *grouped,
                            int window) {
    int len[rd_model::ROWS_MAX];
    for (int b = 0; b < B; b++) len[b] = pos[b] + 1;
    *grouped = build_attn_worklist(len, slot, m->desc.n_heads / m->desc.n_kv_heads, B, m->desc.n_kv_heads, items, ranges, window);
    if ((int)items.size() > m->max_items) {
        rd_set_error("attention work list overflow (%zu items)", items.size());
        return RD_ERR_STATE;
    }
    return RD_OK;
}

// foldW: P holds an MoE layer's down-projection rows and foldW their weights (see the kernel); else split-K partial sums.
// postW: the norm of the pending contribution itself (Gemma 2's post-attention / post-feed-forward norm), or null.
static int add_norm_quant(rd_model *m, float *h, int B, const float *P, int splits, const float *w, const DevWeight &next, void *Xp, float *norm_out,
                          const float *foldW = nullptr, const float *postW = nullptr) {
    rd_device *d = m->d;
    Scope s(m, KC_ADD_NORM);
    return d->launch(d->k.add_rmsnorm_quant, (unsigned)B, 1, 1, 1024, h, P, splits, w, m->desc.rms_eps, m->desc.hidden, Xp, (int)PANEL_A8, norm_out,
                     m->pStride, m->xpAStride, foldW, P ? postW : (const float *)nullptr, act_group_for(next));
}

// One GEMM, or for a group one GEMM per member into column ranges of the same P[split][32][N], all with the group's split
// count so that the consumer sums the same number of partials for every column.
static int launch_proj(rd_model *m, const DevWeight &w, const void *Xp, size_t xpStride, int B, GemmPlan *plan) {
    rd_device *d = m->d;
    if (w.kind != WKIND_GROUP) return launch_gemm_wide(d, w, Xp, xpStride, m->P, m->pStride, B, plan);
    GemmPlan g = group_plan(w);
    for (size_t i = 0; i < w.parts.size(); i++) {
        const DevWeight &p = w.parts[i];
        RC(launch_gemm_wide(d, p, Xp, xpStride, m->P + w.col0[i], m->pStride, B, nullptr, w.N, g.splits));
    }
    g.kbPerSplit = 0;
    if (plan) *plan = g;
    return RD_OK;
}

// Where the fused gate|up kernel can run it sums K over two waves per tile, folded in LDS. The unfused path — steps of more than
// 32 rows, or the fused kernel switched off — is launched with the same two waves and one split, so both produce the same bits
// and a row is the same row in a batch of any size.
static bool gateup_fusable(const rd_model_desc &c, const DevWeight &w) { return w.kind == 0 && c.inter % 32 == 0; }
constexpr int GATEUP_KW = 2; // waves per tile of the fused gate|up kernel

// The q|k|v GEMM can rotate and store its own output where nothing needs a whole head at once: no per-head q/k RMSNorm, the f16
// cache (the int8 cache takes one scale per head), one weight of an int8-MFMA kind (not a group of kinds).
static bool qkv_fusable(const rd_model *m, const LayerW &l) {
    return is_gemm8_kind(l.qkv.kind) && !m->desc.qk_norm && m->kv_type == RD_KV_F16 && !getenv("ROCMDECODE_NO_FUSED_QKV");
}

constexpr int MOE_FOLD_FUSED_MAX = 8; // ranks rd_k_add_rmsnorm_quant folds in registers

static int moe_ffn(rd_model *m, int B, int layer, LayerW &l) {
    rd_device *d = m->d;
    const rd_model_desc &c = m->desc;
    int H = c.hidden, I = c.expert_inter, k = c.top_k, nE = c.n_experts;
    unsigned *bits_dev = m->moe_bits;
    {
        Scope s(m, KC_MOE_ROUTER);
        int *trace = m->moe_idx_all + (size_t)layer * 32 * k;
        if (m->replay_B == B) { // replay a recorded routing (goinfer's moeSelOverride seam) instead of routing on this hidden state
            RC(d->h2d(m->moe_idx, m->replay_idx[(size_t)layer].data(), sizeof(int) * (size_t)B * k));
            RC(d->h2d(m->moe_wgt, m->replay_wgt[(size_t)layer].data(), sizeof(float) * (size_t)B * k));
            RC(d->h2d(m->moe_rank, m->replay_rank[(size_t)layer].data(), (size_t)32 * nE));
            RC(d->h2d(trace, m->replay_idx[(size_t)layer].data(), sizeof(int) * (size_t)B * k));
            unsigned bits[8] = {0, 0, 0, 0, 0, 0, 0, 0}; // the experts the replayed routing uses
            for (int i = 0; i < B * k; i++) {
                int e = m->replay_idx[(size_t)layer][(size_t)i];
                bits[e >> 5] |= 1u << (e & 31);
            }
            RC(d->h2d(bits_dev, bits, sizeof(bits)));
            if (m->moe_rowmax) HIPCHK(MemsetAsync(m->moe_rowmax, 0, sizeof(unsigned) * (size_t)nE * 32, d->stream)); // a replayed step is never captured in a graph
        } else {
            // two launches: the logits over many blocks (one per token would leave the chip idle: measured twice as slow), then the routing
            RC(d->launch(d->k.matmul_f32, (unsigned)((nE + 3) / 4), (unsigned)B, 1, 256, (const float *)m->normed, (const float *)l.router,
                         m->router_logits, B, H, nE, bits_dev, m->moe_rowmax, m->moe_rowmax ? nE * 32 : 0));
            RC(d->launch(d->k.moe_route, (unsigned)B, 1, 1, 64, (const float *)m->router_logits, B, nE, k, c.norm_topk_prob, m->moe_idx, m->moe_wgt,
                         m->moe_rank, trace, bits_dev, (const float *)l.router_bias, m->router_sigmoid, m->router_scale, m->n_group, m->topk_group));
        }
    }
    const int nKBh = (H + 255) / 256, nKBi = (I + 255) / 256;
    size_t guStride = (size_t)(2 * I / 32) * nKBh * 4608, dnStride = (size_t)(H / 32) * nKBi * 4608;
    size_t xpStride = a8_bytes(I);
    const bool rowAct = m->exp_act_group == 0; // one activation scale per row
    const bool fused = I % 32 == 0 && !getenv("ROCMDECODE_NO_FUSED_MOE_GATEUP");
    hipFunction_t gemv = rowAct ? d->k.moe_gemv_w4a8r : d->k.moe_gemv_w4a8;
    if (fused && rowAct) {
        // gate|up + SwiGLU leave f32 rows and their maxima; the per-row quantizer, which needs a whole row, runs where the down projection
        // stages its rows: two launches, as on the per-32 lane
        {
            Scope s(m, KC_MOE_GEMM);
            RC(d->launch_lds(d->k.moe_gemv_w4a8r_gateup, (unsigned)((I / 32 + 1) / 2), (unsigned)nE, moe_pass_layers(B), MOE_THREADS, moe_gemv_lds(H), (const void *)l.exp_gateup, guStride,
                             (const void *)m->XpA, m->XEf, m->moe_rowmax, I, H, B, (const signed char *)m->moe_rank, nE, (const unsigned *)bits_dev));
        }
        Scope s(m, KC_MOE_GEMM_DOWN);
        RC(d->launch_lds(d->k.moe_gemv_w4a8r_f32in, moe_gemv_grid(H, I), (unsigned)nE, 1, MOE_THREADS, moe_gemv_lds(I), (const void *)l.exp_down, dnStride,
                         (const float *)m->XEf, (const unsigned *)m->moe_rowmax, m->moe_dn, H, I, B, k, (const signed char *)m->moe_rank, nE,
                         (const unsigned *)bits_dev));
    } else if (fused) {
        Scope s(m, KC_MOE_GEMM); // gate|up of every touched expert + SwiGLU + quantization into the experts' down activations
        RC(d->launch_lds(d->k.moe_gemv_w4a8_gateup, (unsigned)((I / 32 + 1) / 2), (unsigned)nE, moe_pass_layers(B), MOE_THREADS, moe_gemv_lds(H), (const void *)l.exp_gateup, guStride,
                         (const void *)m->XpA, m->XpE, xpStride, I, H, B, (const signed char *)m->moe_rank, nE, (const unsigned *)bits_dev));
    } else {
        {
            Scope s(m, KC_MOE_GEMM);
            RC(d->launch_lds(gemv, moe_gemv_grid(2 * I, H), (unsigned)nE, moe_pass_layers(B), MOE_THREADS, moe_gemv_lds(H), (const void *)l.exp_gateup, guStride,
                             (const void *)m->XpA, (size_t)0, m->moe_gu, 2 * I, H, B, k, (const signed char *)m->moe_rank, nE,
                             (const unsigned *)bits_dev));
        }
        Scope s(m, KC_MOE_GLUE);
        if (rowAct)
            RC(d->launch(d->k.moe_swiglu_quant_row, (unsigned)(B * k), 1, 1, 256, (const float *)m->moe_gu, (const int *)m->moe_idx, I, k, m->XpE, xpStride,
                         (const signed char *)m->moe_rank, nE));
        else
            RC(d->launch(d->k.moe_swiglu_quant, (unsigned)((I + 255) / 256), (unsigned)(B * k), 1, 256, (const float *)m->moe_gu, (const int *)m->moe_idx,
                         I, k, m->XpE, xpStride, (const signed char *)m->moe_rank, nE));
    }
    if (!(fused && rowAct)) {
        Scope s(m, KC_MOE_GEMM_DOWN);
        RC(d->launch_lds(gemv, moe_gemv_grid(H, I), (unsigned)nE, 1, MOE_THREADS, moe_gemv_lds(I), (const void *)l.exp_down, dnStride,
                         (const void *)m->XpE, xpStride, m->moe_dn, H, I, B, k, (const signed char *)m->moe_rank, nE, (const unsigned *)bits_dev));
    }
    if (k > MOE_FOLD_FUSED_MAX) { // else the next norm kernel folds the ranks itself as it adds them to the residual
        Scope s(m, KC_MOE_GLUE);
        RC(d->launch(d->k.moe_fold, (unsigned)((H + 255) / 256), (unsigned)B, 1, 256, (const float *)m->moe_dn, (const float *)m->moe_wgt, m->moe_out,
                     H, k));
    }
    return RD_OK;
}

// The attention kernel of one layer over the step's work list for it (already on the device): the whole-context list, or the
// sliding-window list for a layer with a window.
int launch_attn_partial(rd_model *m, const LayerW &l) {
    rd_device *d = m->d;
    const rd_model_desc &c = m->desc;
    const int nH = c.n_heads, nKV = c.n_kv_heads, HD = c.head_dim, li = l.window > 0 ? 1 : 0;
    const size_t nItems = m->last_items[li]; // padded to ATTN_LIST_PAD: whole blocks for any of the kernels
    const bool grouped = m->last_grouped[li];
    const void *items = (const int *)m->items + (size_t)li * m->list_ints;
    const AttnLaunch al = attn_partial_kernel(d, m->kv_type == RD_KV_I8, grouped, nItems);
    if (m->kv_type == RD_KV_I8)
        return d->launch(al.f, (unsigned)(nItems / al.waves), 1, 1, 64 * al.waves, items, (const int *)m->rowLen, (const int *)m->rowSlot,
                         (const int *)m->tables, m->blocks_per_slot, (const signed char *)l.Kp, (const signed char *)l.Vp, (const float *)l.Ksc,
                         (const float *)l.Vsc, (const float *)m->qbuf, m->part, nH, nKV, HD, c.attn_scale, c.attn_softcap, l.window);
    return d->launch(al.f, (unsigned)(nItems / al.waves), 1, 1, 64 * al.waves, items, (const int *)m->rowLen, (const int *)m->rowSlot,
                     (const int *)m->tables, m->blocks_per_slot, (const uint16_t *)l.Kp, (const uint16_t *)l.Vp, (const float *)m->qbuf, m->part,
                     nH, nKV, HD, c.attn_scale, c.attn_softcap, l.window);
}

// A step of one row folds its norm-and-quantize launches into the projections that consume them (rd_k_gemm8_q4k_*_norm1: every
// block forms the 16 KB row itself; the same bits, one launch less): where the pending contribution is plain split-K partials
// (or none), the projection is one Q4_K weight quantized per group of 32, and the row fits the kernels' LDS image.
static bool norm1_fusable(const rd_model *m, int B, const DevWeight &next, const float *foldW, const float *postW) {
    const int H = m->desc.hidden;
    return B == 1 && !foldW && !postW && next.kind == 0 && act_group_for(next) == 32 && H % 256 == 0 && H <= 4096 && !getenv("ROCMDECODE_NO_FUSED_NORM");
}

// Every launch of a step between the uploads (metadata, embeddings) and the copies back: the layers, the final norm, the head,
// the argmax. What it launches depends on the model, B, `want`, and the state step_graph_key() lists, and on nothing else: the
// per-step data (positions, tables, work lists, draw records) is read from device memory the uploads have already filled.
static int step_launches(rd_model *m, int B, int want) {
    rd_device *d = m->d;
    const rd_model_desc &c = m->desc;
    const int H = c.hidden, nH = c.n_heads, nKV = c.n_kv_heads, HD = c.head_dim;
    // pending residual contribution: split-K partials of the previous block's last GEMM, or (resW set) an MoE layer's
    // down-projection rows and their weights, folded by the kernel that adds them
    const float *resP = nullptr, *resW = nullptr, *resPost = nullptr; // resPost: the pending contribution's own norm, if any
    int resSplits = 0;
    if (std::any_of(m->layers.begin(), m->layers.end(), [&](const LayerW &l) { return qkv_fusable(m, l); })) {
        Scope s(m, KC_ROPE_STORE);
        RC(d->launch(d->k.rope_table, (unsigned)B, 1, 1, (unsigned)(HD / 2), (const int *)m->rowPos, (const double *)m->inv_freq_dev, m->rope_cs, HD / 2));
    }
    float *h = m->h; // the residual rows; a one-row step alternates between m->h and m->h2 (see norm1_fusable)
    auto other = [&](float *p) { return p == m->h ? m->h2 : m->h; };
    for (int li = 0; li < c.n_layers; li++) {
        LayerW &l = m->layers[(size_t)li];
        GemmPlan plan;
        const bool qkvNorm1 = qkv_fusable(m, l) && gemm8_lane(l.qkv) == 0 && norm1_fusable(m, B, l.qkv, resW, resPost);
        if (!qkvNorm1) RC(add_norm_quant(m, h, B, resP, resSplits, l.attn_norm, l.qkv, m->XpA, nullptr, resW, resPost));
        if (qkvNorm1) {
            Scope s(m, KC_GEMM_QKV); // one row: norm, quantization, projection, bias, RoPE and the KV store in one launch
            const DevWeight &w = l.qkv;
            const int nKB = kblocks_for(w), kw = plan_gemm(w.kind, w.N, nKB, w.act_group).kw;
            RC(d->launch(d->k.gemm8_q4k_qkv_norm1[kw == 8 ? 2 : (kw == 4 ? 1 : 0)], (unsigned)(w.N / 32), 1, 1, (unsigned)(64 * kw), (const void *)w.tiled,
                         (const void *)w.scales, w.N, nKB, m->qbuf, l.Kp, l.Vp, (const int *)m->tables, m->blocks_per_slot, (const int *)m->rowSlot,
                         (const int *)m->rowPos, (const double *)m->rope_cs, (const float *)l.qkv_bias, nH, nKV, HD, (const float *)h, other(h), resP, resSplits,
                         (const float *)l.attn_norm, c.rms_eps, H));
            h = other(h);
        } else if (qkv_fusable(m, l)) {
            Scope s(m, KC_GEMM_QKV); // projection, bias, RoPE and the KV store in one launch (M-tiles of 32 rows as grid.z)
            const DevWeight &w = l.qkv;
            const int nKB = kblocks_for(w), kw = plan_gemm(w.kind, w.N, nKB, w.act_group).kw; // the plain GEMM's waves per tile, in one split
            if (gemm8_lane(w) == 0 && B >= ROWS_GEMM_MIN_ROWS && rows_gemm_enabled()) { // more than 32 rows: four M-tiles per decoded weight tile
                const unsigned gz = (unsigned)((B + 127) / 128);
                const bool two = rows_gemm_two_groups((size_t)(w.N / 32) * gz);
                RC(d->launch(two ? d->k.gemm8_q4k_rows_qkv_g2 : d->k.gemm8_q4k_rows_qkv, (unsigned)(w.N / 32), 1, gz, two ? 512 : 256, (const void *)w.tiled,
                             (const void *)m->XpA, w.N, nKB, kw, B, m->qbuf, l.Kp, l.Vp, (const int *)m->tables, m->blocks_per_slot, (const int *)m->rowSlot,
                             (const int *)m->rowPos, (const double *)m->rope_cs, (const float *)l.qkv_bias, nH, nKV, HD, m->xpAStride));
            } else
            RC(d->launch(d->k.gemm8_qkv[gemm8_lane(w)][kw == 8 ? 2 : (kw == 4 ? 1 : 0)], (unsigned)(w.N / 32), 1, (unsigned)((B + 31) / 32), (unsigned)(64 * kw),
                         (const void *)w.tiled, (const void *)w.scales, (const void *)m->XpA, w.N, nKB, B, m->qbuf, l.Kp, l.Vp, (const int *)m->tables,
                         m->blocks_per_slot, (const int *)m->rowSlot, (const int *)m->rowPos, (const double *)m->rope_cs, (const float *)l.qkv_bias, nH, nKV,
                         HD, m->xpAStride));
        } else {
            {
                Scope s(m, KC_GEMM_QKV);
                RC(launch_proj(m, l.qkv, m->XpA, m->xpAStride, B, &plan));
            }
            Scope s(m, KC_ROPE_STORE);
            if (m->kv_type == RD_KV_I8)
                RC(d->launch(d->k.qkv_rope_store_i8, (unsigned)(nH + 2 * nKV), (unsigned)B, 1, (unsigned)(HD / 2), (const float *)m->P, plan.splits, m->qbuf,
                             (signed char *)l.Kp, (signed char *)l.Vp, l.Ksc, l.Vsc, (const int *)m->tables, m->blocks_per_slot, (const int *)m->rowSlot,
                             (const int *)m->rowPos, (const double *)m->inv_freq_dev, (const float *)l.q_norm, (const float *)l.k_norm, c.rms_eps, nH, nKV,
                             HD, m->pStride, (const float *)l.qkv_bias, 1));
            else
                RC(d->launch(d->k.qkv_rope_store, (unsigned)(nH + 2 * nKV), (unsigned)B, 1, (unsigned)(HD / 2), (const float *)m->P, plan.splits, m->qbuf,
                             l.Kp, l.Vp, (const int *)m->tables, m->blocks_per_slot, (const int *)m->rowSlot, (const int *)m->rowPos,
                             (const double *)m->inv_freq_dev, (const float *)l.q_norm, (const float *)l.k_norm, c.rms_eps, nH, nKV, HD, m->pStride,
                             (const float *)l.qkv_bias, 1));
        }
        {
            Scope s(m, KC_ATTN_PARTIAL);
            if (!m->bench_skip_attn) RC(launch_attn_partial(m, l));
        }
        if (act_group_for(l.o) == 0) {
            // the o projection takes one activation scale per row: the merged heads go out as f32 rows and the per-row quantizer
            // (which needs the whole row's maximum) is its own launch
            Scope s(m, KC_ATTN_COMBINE);
            const int li = l.window > 0 ? 1 : 0;
            RC(d->launch(d->k.attn_combine, (unsigned)nH, (unsigned)B, 1, (unsigned)(ATTN_PIECES * HD / 4), (const float *)m->part,
                         (const int *)m->itemStart + (size_t)li * m->list_ints, m->last_grouped[li] ? ATTN_TILE_ROWS : nH / nKV, m->attn_out, nH, nKV, HD,
                         (const float *)l.sinks));
            for (int r0 = 0; r0 < B; r0 += 32)
                RC(launch_quant_act(d, m->attn_out + (size_t)r0 * nH * HD, std::min(32, B - r0), nH * HD, panel_kind_for(l.o), 0,
                                    (char *)m->XpB + (size_t)(r0 / 32) * m->xpBStride));
        } else {
            Scope s(m, KC_ATTN_COMBINE);
            const int li = l.window > 0 ? 1 : 0;
            RC(d->launch(d->k.attn_combine_quant, (unsigned)nH, (unsigned)B, 1, (unsigned)(ATTN_PIECES * HD / 4), (const float *)m->part,
                         (const int *)m->itemStart + (size_t)li * m->list_ints, m->last_grouped[li] ? ATTN_TILE_ROWS : nH / nKV, m->XpB, panel_kind_for(l.o), nH, nKV,
                         HD, m->xpBStride, (const float *)l.sinks));
        }
        {
            Scope s(m, KC_GEMM_O);
            RC(launch_gemm_wide(d, l.o, m->XpB, m->xpBStride, m->P, m->pStride, B, &plan));
        }
        if (c.n_experts == 0) {
            const bool guFused = gateup_fusable(c, l.gateup) && !getenv("ROCMDECODE_NO_FUSED_GATEUP");
            const bool guNorm1 = guFused && norm1_fusable(m, B, l.gateup, nullptr, l.post_attn_norm);
            if (!guNorm1) RC(add_norm_quant(m, h, B, m->P, plan.splits, l.ffn_norm, l.gateup, m->XpA, nullptr, nullptr, l.post_attn_norm));
            if (guNorm1) {
                Scope s(m, KC_GEMM_GATEUP); // one row: norm, quantization, gate|up, SwiGLU and the down projection's quantization in one launch
                RC(d->launch(m->act == RD_ACT_GELU_TANH ? d->k.gemm8_q4k_gateup_gelu_norm1 : d->k.gemm8_q4k_gateup_norm1, (unsigned)(c.inter / 32), 1, 1,
                             GATEUP_THREADS, (const void *)l.gateup.tiled, m->XpB, panel_kind_for(l.down), c.inter, H / 256, (const float *)h, other(h),
                             (const float *)m->P, plan.splits, (const float *)l.ffn_norm, c.rms_eps, H));
                h = other(h);
            } else if (guFused) {
                Scope s(m, KC_GEMM_GATEUP); // gate|up GEMM + SwiGLU + quantization in one launch (M-tiles of 32 rows as grid.z)
                if (B >= ROWS_GEMM_MIN_ROWS && rows_gemm_enabled()) // more than 32 rows: four M-tiles per decoded weight tile
                    RC(d->launch(m->act == RD_ACT_GELU_TANH ? d->k.gemm8_q4k_rows_gateup_gelu : d->k.gemm8_q4k_rows_gateup, (unsigned)(c.inter / 32), 1,
                                 (unsigned)((B + 127) / 128), 256, (const void *)l.gateup.tiled, (const void *)m->XpA, m->XpB, c.inter, H / 256, B, m->xpAStride,
                                 m->xpBStride));
                else
                RC(d->launch(m->act == RD_ACT_GELU_TANH ? d->k.gemm8_q4k_gateup_gelu : d->k.gemm8_q4k_gateup, (unsigned)(c.inter / 32), 1, (unsigned)((B + 31) / 32), GATEUP_THREADS, (const void *)l.gateup.tiled,
                             (const void *)m->XpA, m->XpB, panel_kind_for(l.down), c.inter, H / 256, B, m->xpAStride, m->xpBStride));
            } else {
                {
                    Scope s(m, KC_GEMM_GATEUP);
                    if (gateup_fusable(c, l.gateup))
                        RC(launch_gemm_wide(d, l.gateup, m->XpA, m->xpAStride, m->P, m->pStride, B, &plan, 0, 1, GATEUP_KW));
                    else
                        RC(launch_proj(m, l.gateup, m->XpA, m->xpAStride, B, &plan));
                }
                Scope s(m, KC_SWIGLU);
                if (act_group_for(l.down) == 0)
                    RC(d->launch(d->k.swiglu_quant_row, (unsigned)B, 1, 1, 1024, (const float *)m->P, plan.splits, c.inter, m->XpB, panel_kind_for(l.down),
                                 m->pStride, m->xpBStride, m->act));
                else
                    RC(d->launch(d->k.swiglu_quant, (unsigned)((c.inter + 1023) / 1024), (unsigned)B, 1, 256, (const float *)m->P, plan.splits, c.inter,
                                 m->XpB, panel_kind_for(l.down), (float *)nullptr, m->pStride, m->xpBStride, m->act));
            }
            {
                Scope s(m, KC_GEMM_DOWN);
                RC(launch_gemm_wide(d, l.down, m->XpB, m->xpBStride, m->P, m->pStride, B, &plan));
            }
            resP = m->P, resSplits = plan.splits, resW = nullptr, resPost = l.post_ffn_norm;
        } else {
            {
                Scope s(m, KC_ADD_NORM);
                RC(d->launch(d->k.add_rmsnorm_quant, (unsigned)B, 1, 1, 1024, h, (const float *)m->P, plan.splits, (const float *)l.ffn_norm,
                             c.rms_eps, H, m->XpA, (int)PANEL_ROW8, m->normed, m->pStride, m->xpAStride, (const float *)nullptr,
                             (const float *)nullptr, m->exp_act_group == 0 ? 0 : 32));
            }
            RC(moe_ffn(m, B, li, l));
            if (c.top_k <= MOE_FOLD_FUSED_MAX)
                resP = m->moe_dn, resSplits = c.top_k, resW = m->moe_wgt, resPost = nullptr;
            else
                resP = m->moe_out, resSplits = 1, resW = nullptr, resPost = nullptr;
        }
    }
    if (want & (RD_WANT_LOGITS | RD_WANT_ARGMAX)) {
        GemmPlan plan;
        RC(add_norm_quant(m, h, B, resP, resSplits, m->final_norm, m->head, m->XpA, nullptr, resW, resPost));
        {
            Scope s(m, KC_GEMM_HEAD);
            RC(launch_gemm_wide(d, m->head, m->XpA, m->xpAStride, m->P, m->pStride, B, &plan));
        }
        {
            Scope s(m, KC_ARGMAX);
            int nChunks = (c.vocab + 4095) / 4096;
            RC(d->launch(d->k.argmax_rows, (unsigned)nChunks, (unsigned)B, 1, 256, (const float *)m->P, plan.splits, c.vocab, m->cand_v, m->cand_i,
                         (want & RD_WANT_LOGITS) ? m->logits : (float *)nullptr, (const int *)(m->step_draws ? m->rowDraw : nullptr), m->pStride,
                         m->final_softcap, m->logit_mul));
            if (want & RD_WANT_ARGMAX) RC(d->launch(d->k.argmax_final, (unsigned)B, 1, 1, 64, (const float *)m->cand_v, (const int *)m->cand_i, nChunks, m->ids));
        }
    }
    return RD_OK;
}

// What step_launches() reads besides the model: two steps with equal keys issue the same launches with the same arguments, so
// the second may replay the first one's captured graph. Empty: this step is not one to capture (timed, or replaying a routing).
static std::vector<long> step_graph_key(rd_model *m, int B, int want) {
    std::vector<long> k;
    if (m->timer.on || m->replay_B != 0 || m->bench_skip_attn) return k;
    k = {B, want, m->step_draws ? 1 : 0, (long)m->last_items[0], (long)m->last_items[1], m->last_grouped[0] ? 1 : 0, m->last_grouped[1] ? 1 : 0};
    // every environment knob a launch consults, by value: a step after a change is launched (and captured) anew
    for (const char *name : {"ROCMDECODE_NO_FUSED_GATEUP", "ROCMDECODE_NO_FUSED_QKV", "ROCMDECODE_NO_FUSED_MOE_GATEUP", "ROCMDECODE_MOE_TILES",
                             "ROCMDECODE_GEMM8_KW", "ROCMDECODE_GEMM8_SPLITS", "ROCMDECODE_NO_DEEP_ATTN", "ROCMDECODE_NO_WIDE_ATTN",
                             "ROCMDECODE_NO_ATTN_GROUPS", "ROCMDECODE_NO_ROWS_GEMM", "ROCMDECODE_NO_FUSED_NORM", "ROCMDECODE_MOE_PASS_LAYERS"}) {
        const char *e = getenv(name);
        k.push_back(e ? 1 + atol(e) : 0);
    }
    return k;
}

static void step_graph_drop(rd_model *m) {
    rd_device *d = m->d;
    if (m->graph.exec) (void)d->hip->GraphExecDestroy(m->graph.exec);
    if (m->graph.graph) (void)d->hip->GraphDestroy(m->graph.graph);
    m->graph.exec = nullptr, m->graph.graph = nullptr, m->graph.key.clear();
}

// The launches of a step, from a captured HIP graph when this step repeats the previous one's key (a decode loop whose work list
// keeps its size: every step of a batch between two piece boundaries), eagerly otherwise. The second step in a row with one key
// is captured (stream capture records the launches without running them) and the graph, once instantiated, runs that step too.
// Any failure of the graph calls ends graph use for this model and the step is launched eagerly: the result is the same bits.
static int step_run(rd_model *m, int B, int want) {
    rd_device *d = m->d;
    const HipApi *hip = d->hip;
    std::vector<long> key;
    if (m->graph.enabled) key = step_graph_key(m, B, want);
    if (key.empty()) {
        m->graph.prev_key.clear();
        return step_launches(m, B, want);
    }
    if (m->graph.exec && key == m->graph.key) {
        if (rd_hip_ok(hip, hip->GraphLaunch(m->graph.exec, d->stream), "hipGraphLaunch")) {
            m->graph.replays++;
            return RD_OK;
        }
        m->graph.enabled = false; // nothing of this step has run: fall through to the eager launches
        step_graph_drop(m);
        return step_launches(m, B, want);
    }
    const bool repeat = key == m->graph.prev_key;
    m->graph.prev_key = key;
    if (!repeat) return step_launches(m, B, want);
    step_graph_drop(m);
    if (!rd_hip_ok(hip, hip->StreamBeginCapture(d->stream, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture")) {
        m->graph.enabled = false;
        return step_launches(m, B, want);
    }
    const int rc = step_launches(m, B, want);
    hipGraph_t g = nullptr;
    const bool ended = rd_hip_ok(hip, hip->StreamEndCapture(d->stream, &g), "hipStreamEndCapture");
    if (rc || !ended || !g || !rd_hip_ok(hip, hip->GraphInstantiate(&m->graph.exec, g, nullptr, nullptr, 0), "hipGraphInstantiate")) {
        if (g) (void)hip->GraphDestroy(g);
        m->graph.exec = nullptr, m->graph.enabled = false;
        return rc ? rc : step_launches(m, B, want); // the capture ran nothing
    }
    m->graph.graph = g, m->graph.key = key, m->graph.captures++;
    if (rd_hip_ok(hip, hip->GraphLaunch(m->graph.exec, d->stream), "hipGraphLaunch")) return RD_OK;
    m->graph.enabled = false;
    step_graph_drop(m);
    return step_launches(m, B, want);
}

// Graph replay of the step's launches on or off (on at creation unless ROCMDECODE_NO_GRAPH is set), and how often it was used.
extern "C" int rd_model_set_graph(rd_model *m, int on) {
    if (!m) return RD_ERR_ARG;
    RC(m->d->sync());
    step_graph_drop(m);
    m->graph.prev_key.clear();
    m->graph.enabled = false;
    if (on && !graph_allowed()) {
        rd_set_error("graph replay stays off: a profiler tool library is attached (ROCP_TOOL_LIBRARIES); ROCMDECODE_GRAPH=1 overrides");
        return RD_DECLINED;
    }
    m->graph.enabled = on != 0;
    return RD_OK;
}

extern "C" int rd_model_graph_stats(rd_model *m, long long *captures, long long *replays) {
    if (!m) return RD_ERR_ARG;
    if (captures) *captures = m->graph.captures;
    if (replays) *replays = m->graph.replays;
    return RD_OK;
}

// emb_host: [B][hidden] on the host, or emb_dev already on the device (benchmark loop). Logits/ids are host pointers.
int model_step(rd_model *m, int B, const int *slot, const int *pos, const float *emb_host, const float *emb_dev, int want, float *logits,
               int *ids, bool multirow) {
    rd_device *d = m->d;
    const rd_model_desc &c = m->desc;
    if (!m->finalized || !m->tables) {
        rd_set_error("step before rd_model_finalize / rd_kv_configure");
        return RD_ERR_STATE;
    }
    if (m->chain.open && !m->chain.in_call) {
        rd_set_error("a chain is open: between its start and stop the resident takes no other step");
        return RD_ERR_STATE;
    }
    if (B < 1 || B > m->max_rows) {
        rd_set_error("rocm resident: batch %d outside the stepper range 1..%d", B, m->max_rows);
        return RD_ERR_ARG;
    }
    RC(d->use());
    // A slot may carry several rows in one step if they sit at consecutive positions (a ragged step's verify or prefill
    // rows): all their K/V is written before any row attends, and row j reads keys [0, pos_j], so each row is the row its own
    // single-token step would compute. Anything else naming a slot twice is refused before a byte is written.
    for (int b = 0; b < B; b++) {
        if (!slot_ok(m, slot[b])) return RD_ERR_ARG;
        int prev = -1;
        for (int a = 0; a < b; a++)
            if (slot[a] == slot[b]) prev = a;
        if (prev >= 0) {
            if (!multirow || pos[b] != pos[prev] + 1) {
                rd_set_error("slot %d appears twice in one step", slot[b]);
                return RD_ERR_ARG;
            }
        } else if (pos[b] < 0 || pos[b] > m->slot_len[(size_t)slot[b]]) {
            rd_set_error("row %d: position %d but slot %d holds %d rows", b, pos[b], slot[b], m->slot_len[(size_t)slot[b]]);
            return RD_ERR_ARG;
        }
        if (pos[b] >= m->ctx_cap) { // ErrKVPoolFull: nothing has been written
            rd_set_error("row %d: position %d reaches the context cap %d", b, pos[b], m->ctx_cap);
            return RD_ERR_KV_FULL;
        }
    }
    const int H = c.hidden, nKV = c.n_kv_heads;
    const int nLists = m->window > 0 ? 2 : 1;
    std::vector<AttnItemH> items[2];
    std::vector<int> start[2];
    for (int li = 0; li < nLists; li++) {
        bool grouped = false;
        RC(build_attn_items(m, B, slot, pos, items[li], start[li], &grouped, li ? m->window : 0));
        // The list is launched padded to a multiple of ATTN_LIST_PAD with items that name no row (their waves leave at once):
        // the launch then keeps its shape over many steps of a growing batch, which is what lets a captured graph be replayed.
        attn_pad_items(items[li]);
        m->last_items[li] = items[li].size(), m->last_grouped[li] = grouped;
    }
    // Stage the step's metadata (and host embeddings) in pinned memory and upload it asynchronously. A slot is reused only
    // once the upload it last fed has completed, which its event tells.
    const unsigned stage_slot = m->stage_next++ % rd_model::STAGE_SLOTS;
    if (m->stage_busy[stage_slot]) HIPCHK(EventSynchronize(m->stage_ev[stage_slot]));
    {
        char *st = (char *)m->host_stage + (size_t)stage_slot * m->host_stage_bytes;
        int *hm = (int *)st; // the metadata block, laid out as on the device
        const size_t rangeInts = (size_t)m->max_rows * nKV * ATTN_RANGE_INTS;
        constexpr int RM = rd_model::ROWS_MAX;
        float *eh = (float *)(st + m->stage_meta_bytes);
        for (int b = 0; b < B; b++) hm[b] = slot[b], hm[RM + b] = pos[b], hm[2 * RM + b] = pos[b] + 1;
        // Draw records (resident/forward.go:43-52 BatchDraw) with Sampler.gumbelDraw's guards applied here
        // (internal/runtime/sampling/sampler_gumbel.go:80-88): a temperature <= 0 means 1, and one so small that 1/T
        // overflows f32 is the plain argmax.
        for (int b = 0; b < RM; b++) {
            int *r = hm + 3 * RM + b * 6;
            memset(r, 0, sizeof(int) * 6);
            if (b >= B || !m->step_draws) continue;
            const rd_draw &dw = m->step_draws[b];
            r[0] = dw.mode;
            if (dw.mode == RD_DRAW_GUMBEL) {
                float invT = (float)(1.0 / (dw.temperature <= 0 ? 1.0 : dw.temperature));
                if (std::isinf(invT)) {
                    r[0] = RD_DRAW_GREEDY;
                    continue;
                }
                memcpy(&r[1], &invT, 4);
                r[2] = (int)(uint32_t)dw.seed, r[3] = (int)(uint32_t)(dw.seed >> 32);
                r[4] = (int)(uint32_t)dw.draw, r[5] = (int)(uint32_t)(dw.draw >> 32);
            }
        }
        constexpr int HDR = rd_model::META_HDR;
        memset(hm + HDR - 8, 0, sizeof(int) * 8);
        for (int li = 0; li < nLists; li++) {
            int *lst = hm + HDR + (size_t)li * m->list_ints;
            memcpy(lst, start[li].data(), sizeof(int) * start[li].size());
            memcpy(lst + rangeInts, items[li].data(), sizeof(AttnItemH) * items[li].size());
        }
        RC(d->h2d(m->meta, hm, sizeof(int) * (HDR + (size_t)(nLists - 1) * m->list_ints + rangeInts + items[nLists - 1].size() * 4)));
        if (emb_host) {
            memcpy(eh, emb_host, sizeof(float) * (size_t)B * H);
            RC(d->h2d(m->h, eh, sizeof(float) * (size_t)B * H));
        }
        HIPCHK(EventRecord(m->stage_ev[stage_slot], d->stream));
        m->stage_busy[stage_slot] = true;
        if (emb_host) {
        } else if (emb_dev) {
            HIPCHK(MemcpyAsync(m->h, emb_dev, sizeof(float) * (size_t)B * H, hipMemcpyDeviceToDevice, d->stream));
        } else { // greedy chain: the previous step's argmax ids, still on the device
            if (!m->embed_q) {
                rd_set_error("greedy chain needs rd_model_upload_embedding");
                return RD_ERR_STATE;
            }
            RC(d->launch(d->k.embed_rows, (unsigned)B, 1, 1, 256, (const signed char *)m->embed_q, (const float *)m->embed_scale, (const int *)m->ids,
                         m->h, H));
        }
    }
    RC(step_run(m, B, want));
    // else: no logits asked for (resident.Forward's ForwardNoLogits, decoder/resident/subsystems.go:68-77: a prompt token that only
    // builds its K/V): the final norm, the head GEMM and the argmax are skipped, and the last block's pending residual
    // contribution stays unadded, since nothing reads the hidden state after it.
    for (int b = 0; b < B; b++) m->slot_len[(size_t)slot[b]] = std::max(m->slot_len[(size_t)slot[b]], pos[b] + 1);
    m->last_B = B;
    m->last_logits_valid = (want & RD_WANT_LOGITS) != 0;
    const bool replayed = m->replay_B != 0;
    m->replay_B = 0; // a routing override lasts one step
    if (replayed) RC(d->sync()); // its host arrays were uploaded from pageable memory: let the copies finish before they can change
    if ((want & RD_WANT_LOGITS) && logits) RC(d->d2h(logits, m->logits, sizeof(float) * (size_t)B * c.vocab));
    if ((want & RD_WANT_ARGMAX) && ids) RC(d->d2h(ids, m->ids, sizeof(int) * (size_t)B));
    return RD_OK;
}

extern "C" int rd_model_max_rows(const rd_model *m) { return m && m->finalized ? m->max_rows : 0; }

extern "C" int rd_step_batch(rd_model *m, int B, const int *slot, const int *pos, const float *emb, int want, float *logits, int *ids) {
    if (!m || !slot || !pos || !emb) return RD_ERR_ARG;
    if (((want & RD_WANT_LOGITS) && !logits) || ((want & RD_WANT_ARGMAX) && !ids) || !(want & 3)) {
        rd_set_error("rd_step_batch: want=%d needs its output buffer", want);
        return RD_ERR_ARG;
    }
    return model_step(m, B, slot, pos, emb, nullptr, want, logits, ids, false);
}

// ---------------------------------------------------------------- device-chained decode
// decoder/resident/subsystems.go:78-100: GreedyChainStart / GreedyChainNext / GreedyChainStop and their temperature-only
// siblings SampleChainStart / SampleChainNext. Each forward takes its input row from the embedding table at the id the previous
// forward picked, all on the device; the host reads four bytes per token and the next forward is already queued when it does.
static int chain_queue(rd_model *m) {
    rd_model::Chain &ch = m->chain;
    rd_device *d = m->d;
    rd_draw dw{};
    dw.mode = ch.sample ? RD_DRAW_GUMBEL : RD_DRAW_GREEDY;
    dw.temperature = ch.temperature, dw.seed = ch.seed, dw.draw = ch.draw_next;
    m->step_draws = &dw;
    ch.in_call = true;
    int rc = model_step(m, 1, &ch.slot, &ch.next_pos, nullptr, nullptr, RD_WANT_ARGMAX, nullptr, nullptr, false);
    ch.in_call = false;
    m->step_draws = nullptr;
    if (rc) return rc;
    unsigned s = ch.tail % rd_model::Chain::DEPTH;
    HIPCHK(MemcpyAsync(ch.host_ids + s, m->ids, sizeof(int), hipMemcpyDeviceToHost, d->stream));
    HIPCHK(EventRecord(ch.ev[s], d->stream));
    ch.tail++, ch.next_pos++, ch.draw_next++;
    return RD_OK;
}

// Queue ahead; a look-ahead forward that cannot run (the context cap) is not an error until its token is asked for.
static void chain_look_ahead(rd_model *m) {
    rd_model::Chain &ch = m->chain;
    while (!ch.exhausted && ch.tail - ch.head < (unsigned)rd_model::Chain::DEPTH) {
        int rc = chain_queue(m);
        if (rc) ch.exhausted = true, ch.exhausted_rc = rc;
    }
}

static int chain_start(rd_model *m, int slot, int id, int pos, bool sample, double temperature, uint64_t seed, uint64_t draw) {
    if (!m) return RD_ERR_ARG;
    rd_model::Chain &ch = m->chain;
    if (ch.open) {
        rd_set_error("a chain is already open");
        return RD_ERR_STATE;
    }
    if (!m->finalized || !m->tables || !m->embed_q) {
        rd_set_error("a chain needs rd_model_finalize, rd_kv_configure and rd_model_upload_embedding");
        return RD_ERR_STATE;
    }
    if (id < 0 || id >= m->desc.vocab || !slot_ok(m, slot)) {
        rd_set_error("chain start: token %d or slot %d out of range", id, slot);
        return RD_ERR_ARG;
    }
    rd_device *d = m->d;
    RC(d->use());
    if (!ch.host_ids) {
        HIPCHK(HostMalloc((void **)&ch.host_ids, sizeof(int) * rd_model::Chain::DEPTH, 0));
        for (auto &e : ch.ev) HIPCHK(EventCreate(&e));
    }
    RC(d->h2d(m->ids, &id, sizeof(int)));
    ch.slot = slot, ch.next_pos = pos, ch.sample = sample, ch.temperature = temperature, ch.seed = seed;
    ch.draw_next = ch.draw_head = draw, ch.head = ch.tail = 0, ch.exhausted = false, ch.exhausted_rc = 0;
    int rc = chain_queue(m); // the first forward's own failure (bad position, context cap) is the caller's
    if (rc) return rc;
    ch.open = true;
    chain_look_ahead(m);
    return RD_OK;
}

static int chain_next(rd_model *m, int *id) {
    if (!m || !id) return RD_ERR_ARG;
    rd_model::Chain &ch = m->chain;
    if (!ch.open) {
        rd_set_error("no chain is open");
        return RD_ERR_STATE;
    }
    if (ch.head == ch.tail) { // nothing queued: the look-ahead had failed
        rd_set_error("chain: the forward at position %d could not be queued (%d)", ch.next_pos, ch.exhausted_rc);
        return ch.exhausted_rc ? ch.exhausted_rc : RD_ERR_STATE;
    }
    unsigned s = ch.head % rd_model::Chain::DEPTH;
    rd_device *d = m->d;
    HIPCHK(EventSynchronize(ch.ev[s]));
    *id = ch.host_ids[s];
    ch.head++, ch.draw_head++;
    chain_look_ahead(m);
    return RD_OK;
}

extern "C" int rd_greedy_chain_start(rd_model *m, int slot, int id, int pos) { return chain_start(m, slot, id, pos, false, 1.0, 0, 0); }
extern "C" int rd_greedy_chain_next(rd_model *m, int *id) {
    if (m && m->chain.open && m->chain.sample) {
        rd_set_error("the open chain is a sample chain");
        return RD_ERR_STATE;
    }
    return chain_next(m, id);
}
extern "C" int rd_sample_chain_start(rd_model *m, int slot, int id, int pos, double temperature, uint64_t seed, uint64_t draw) {
    if (std::isnan(temperature)) return RD_ERR_ARG;
    return chain_start(m, slot, id, pos, true, temperature, seed, draw);
}
extern "C" int rd_sample_chain_next(rd_model *m, uint64_t seed, uint64_t draw, int *id) {
    if (!m) return RD_ERR_ARG;
    rd_model::Chain &ch = m->chain;
    if (!ch.open || !ch.sample) {
        rd_set_error("no sample chain is open");
        return RD_ERR_STATE;
    }
    if (seed != ch.seed || draw != ch.draw_head) { // the caller's sampler and the chain must agree on the draw of this forward
        rd_set_error("sample chain: the forward was drawn with (seed %llu, draw %llu), not (%llu, %llu)", (unsigned long long)ch.seed,
                     (unsigned long long)ch.draw_head, (unsigned long long)seed, (unsigned long long)draw);
        return RD_ERR_ARG;
    }
    return chain_next(m, id);
}
// Waits out any forward queued past the last token taken. Those forwards have written their K/V rows (the rows of tokens the
// chain itself picked); positions at or past the one the caller continues from are simply written again.
extern "C" void rd_greedy_chain_stop(rd_model *m) {
    if (!m || !m->chain.open) return;
    (void)m->d->sync();
    m->chain.open = false;
}

// StepBatch with per-row draws (resident/forward.go:37-58): a row with a draw returns the id drawn on the device — the argmax
// for a greedy draw, the Gumbel-max token for a temperature draw — and a row without one returns -1 in ids.
extern "C" int rd_step_batch_draw(rd_model *m, int B, const int *slot, const int *pos, const float *emb, const rd_draw *draws, int want,
                                  float *logits, int *ids) {
    if (!m || !slot || !pos || !emb || !draws || !ids) return RD_ERR_ARG;
    if ((want & RD_WANT_LOGITS) && !logits) {
        rd_set_error("rd_step_batch_draw: want=%d needs its output buffer", want);
        return RD_ERR_ARG;
    }
    for (int b = 0; b < B && b < m->max_rows; b++)
        if (draws[b].mode < RD_DRAW_NONE || draws[b].mode > RD_DRAW_GUMBEL || (draws[b].mode == RD_DRAW_GUMBEL && std::isnan(draws[b].temperature))) {
            rd_set_error("rd_step_batch_draw: row %d has draw mode %d, temperature %g", b, draws[b].mode, draws[b].temperature);
            return RD_ERR_ARG;
        }
    m->step_draws = draws;
    int rc = model_step(m, B, slot, pos, emb, nullptr, want | RD_WANT_ARGMAX, logits, ids, false);
    m->step_draws = nullptr;
    if (!rc)
        for (int b = 0; b < B; b++)
            if (draws[b].mode == RD_DRAW_NONE) ids[b] = -1;
    return rc;
}

// resident/subsystems.go:112-117 StepRagged, forward.go:9-16 ForwardN, subsystems.go:124 PrefillLast: sequences of one or more
// rows at consecutive positions. Rows go through the step's kernels in passes of at most 128 (four GEMM row tiles; 32 for a MoE model), in the
// order given; a sequence longer than a pass simply continues in the next one.
extern "C" int rd_step_ragged(rd_model *m, int n_seq, const int *slot, const int *pos, const int *n_rows, const float *emb, int want, float *logits,
                              int *ids) {
    if (!m || !slot || !pos || !n_rows || !emb || n_seq <= 0) return RD_ERR_ARG;
    if (((want & RD_WANT_LOGITS) && !logits) || ((want & RD_WANT_ARGMAX) && !ids) || !(want & 3)) {
        rd_set_error("rd_step_ragged: want=%d needs its output buffer", want);
        return RD_ERR_ARG;
    }
    if (!m->finalized || !m->tables) {
        rd_set_error("step before rd_model_finalize / rd_kv_configure");
        return RD_ERR_STATE;
    }
    // validate the whole call first: a refused call writes nothing
    std::vector<int> rslot, rpos;
    for (int i = 0; i < n_seq; i++) {
        if (!slot_ok(m, slot[i])) return RD_ERR_ARG;
        for (int a = 0; a < i; a++)
            if (slot[a] == slot[i]) {
                rd_set_error("KV slot %d is named by two sequences", slot[i]);
                return RD_ERR_ARG;
            }
        if (n_rows[i] <= 0) {
            rd_set_error("sequence %d has no rows", i);
            return RD_ERR_ARG;
        }
        if (pos[i] < 0 || pos[i] > m->slot_len[(size_t)slot[i]]) {
            rd_set_error("sequence %d: position %d but slot %d holds %d rows", i, pos[i], slot[i], m->slot_len[(size_t)slot[i]]);
            return RD_ERR_ARG;
        }
        if (pos[i] + n_rows[i] > m->ctx_cap) {
            rd_set_error("sequence %d: rows %d..%d reach the context cap %d", i, pos[i], pos[i] + n_rows[i] - 1, m->ctx_cap);
            return RD_ERR_KV_FULL;
        }
        for (int j = 0; j < n_rows[i]; j++) rslot.push_back(slot[i]), rpos.push_back(pos[i] + j);
    }
    const size_t H = (size_t)m->desc.hidden, V = (size_t)m->desc.vocab;
    const size_t pass = (size_t)m->max_rows; // rows per pass: the step's widest batch
    for (size_t r0 = 0; r0 < rslot.size(); r0 += pass) {
        const int rows = (int)std::min<size_t>(pass, rslot.size() - r0);
        RC(model_step(m, rows, rslot.data() + r0, rpos.data() + r0, emb + r0 * H, nullptr, want, logits ? logits + r0 * V : nullptr,
                      ids ? ids + r0 : nullptr, true));
    }
    return RD_OK;
}

// StepRagged with a draw per sequence (decoder/resident/forward.go:60-75 RaggedSeq.Draw): the last row of a sequence that carries a
// draw returns the token drawn on the device in ids; every other row returns -1 there.
extern "C" int rd_step_ragged_draw(rd_model *m, int n_seq, const int *slot, const int *pos, const int *n_rows, const float *emb, const rd_draw *draws,
                                   int want, float *logits, int *ids) {
    if (!m || !slot || !pos || !n_rows || !emb || !draws || !ids || n_seq <= 0) return RD_ERR_ARG;
    if ((want & RD_WANT_LOGITS) && !logits) {
        rd_set_error("rd_step_ragged_draw: want=%d needs its output buffer", want);
        return RD_ERR_ARG;
    }
    if (!m->finalized || !m->tables) {
        rd_set_error("step before rd_model_finalize / rd_kv_configure");
        return RD_ERR_STATE;
    }
    std::vector<int> rslot, rpos;
    std::vector<rd_draw> rdraw;
    for (int i = 0; i < n_seq; i++) {
        if (!slot_ok(m, slot[i])) return RD_ERR_ARG;
        for (int a = 0; a < i; a++)
            if (slot[a] == slot[i]) {
                rd_set_error("KV slot %d is named by two sequences", slot[i]);
                return RD_ERR_ARG;
            }
        if (n_rows[i] <= 0 || pos[i] < 0 || pos[i] > m->slot_len[(size_t)slot[i]]) {
            rd_set_error("sequence %d: %d rows at position %d, slot %d holds %d rows", i, n_rows[i], pos[i], slot[i], m->slot_len[(size_t)slot[i]]);
            return RD_ERR_ARG;
        }
        if (pos[i] + n_rows[i] > m->ctx_cap) {
            rd_set_error("sequence %d: rows %d..%d reach the context cap %d", i, pos[i], pos[i] + n_rows[i] - 1, m->ctx_cap);
            return RD_ERR_KV_FULL;
        }
        if (draws[i].mode < RD_DRAW_NONE || draws[i].mode > RD_DRAW_GUMBEL || (draws[i].mode == RD_DRAW_GUMBEL && std::isnan(draws[i].temperature))) {
            rd_set_error("rd_step_ragged_draw: sequence %d has draw mode %d, temperature %g", i, draws[i].mode, draws[i].temperature);
            return RD_ERR_ARG;
        }
        for (int j = 0; j < n_rows[i]; j++) {
            rslot.push_back(slot[i]), rpos.push_back(pos[i] + j);
            rd_draw none{};
            rdraw.push_back(j == n_rows[i] - 1 ? draws[i] : none);
        }
    }
    const size_t H = (size_t)m->desc.hidden, V = (size_t)m->desc.vocab;
    int rc = RD_OK;
    const size_t pass = (size_t)m->max_rows;
    for (size_t r0 = 0; r0 < rslot.size() && !rc; r0 += pass) {
        const int rows = (int)std::min<size_t>(pass, rslot.size() - r0);
        m->step_draws = rdraw.data() + r0;
        rc = model_step(m, rows, rslot.data() + r0, rpos.data() + r0, emb + r0 * H, nullptr, want | RD_WANT_ARGMAX, logits ? logits + r0 * V : nullptr,
                        ids + r0, true);
        m->step_draws = nullptr;
    }
    if (!rc)
        for (size_t r = 0; r < rslot.size(); r++)
            if (rdraw[r].mode == RD_DRAW_NONE) ids[r] = -1;
    return rc;
}

// ForwardNoLogits (decoder/resident/subsystems.go:68-77): one token's forward that only builds its K/V; the layer chain, hence the
// K/V written, is the one rd_forward runs.
extern "C" int rd_forward_no_logits(rd_model *m, int slot, int pos, const float *emb) {
    if (!m || !emb) return RD_ERR_ARG;
    return model_step(m, 1, &slot, &pos, emb, nullptr, 0, nullptr, nullptr, false);
}

// PrefillLast: n rows of one sequence from start_pos; only the last row's logits come back.
extern "C" int rd_prefill_last(rd_model *m, int slot, int start_pos, int n, const float *emb, float *logits) {
    if (!m || !emb || !logits || n <= 0) return RD_ERR_ARG;
    if (!m->finalized || !m->tables) {
        rd_set_error("prefill before rd_model_finalize / rd_kv_configure");
        return RD_ERR_STATE;
    }
    if (!slot_ok(m, slot)) return RD_ERR_ARG;
    if (start_pos < 0 || start_pos > m->slot_len[(size_t)slot]) {
        rd_set_error("prefill at position %d but slot %d holds %d rows", start_pos, slot, m->slot_len[(size_t)slot]);
        return RD_ERR_ARG;
    }
    if (start_pos + n > m->ctx_cap) {
        rd_set_error("prefill rows %d..%d reach the context cap %d", start_pos, start_pos + n - 1, m->ctx_cap);
        return RD_ERR_KV_FULL;
    }
    const size_t H = (size_t)m->desc.hidden;
    // All rows but the last only build their K/V (no final norm, no head, nothing read back), in passes as wide as the step
    // takes; the last row is an ordinary one-row step whose logits are the answer. Each row is the row its own single-token
    // forward computes, whatever pass it rides in.
    const int pass = m->max_rows;
    std::vector<int> rslot((size_t)pass, slot), rpos((size_t)pass);
    for (int r0 = 0; r0 < n - 1; r0 += pass) {
        const int rows = std::min(pass, n - 1 - r0);
        for (int j = 0; j < rows; j++) rpos[(size_t)j] = start_pos + r0 + j;
        RC(model_step(m, rows, rslot.data(), rpos.data(), emb + (size_t)r0 * H, nullptr, 0, nullptr, nullptr, true));
    }
    const int lastPos = start_pos + n - 1;
    RC(model_step(m, 1, &slot, &lastPos, emb + (size_t)(n - 1) * H, nullptr, RD_WANT_LOGITS, logits, nullptr, false));
    return RD_OK;
}

extern "C" int rd_forward(rd_model *m, int slot, int pos, const float *emb, float *logits) {
    if (!m || !emb || !logits) return RD_ERR_ARG;
    return model_step(m, 1, &slot, &pos, emb, nullptr, RD_WANT_LOGITS, logits, nullptr, false);
}

// resident.TopKRow (decoder/resident/forward.go:86-96; ForwardTopK, backend/cuda/topk.go:30-67): the step's kernel chain, then
// each row's logits reduced on the device to its k best entries; k*8 bytes (+8 for Z) per row come back instead of vocab*4.
extern "C" int rd_step_batch_topk(rd_model *m, int B, const int *slot, const int *pos, const float *emb, int k, const double *temperature,
                                  int want_z, int *ids, float *vals, double *z) {
    if (!m || !slot || !pos || !emb || !ids || !vals || (want_z && (!z || !temperature))) return RD_ERR_ARG;
    if (k < 1 || k > TOPK_MAX) {
        rd_set_error("rd_step_batch_topk: k=%d outside [1,%d]", k, TOPK_MAX);
        return RD_ERR_ARG;
    }
    rd_device *d = m->d;
    const int V = m->desc.vocab;
    if (k > V) k = V;
    RC(model_step(m, B, slot, pos, emb, nullptr, RD_WANT_LOGITS, nullptr, nullptr, false)); // the logits stay on the device
    if (want_z) {
        float invT[rd_model::ROWS_MAX];
        for (int b = 0; b < B; b++) invT[b] = temperature[b] > 0 ? (float)(1.0 / temperature[b]) : 1.f; // backend/cuda/topk.go:74-77
        RC(d->h2d(m->topk_scratch.invT, invT, sizeof(float) * (size_t)B));
    }
    RC(launch_topk(d, (const float *)m->logits, B, V, k, 1.f, want_z != 0, m->topk_scratch, m->topk_ids, m->topk_vals,
                   want_z ? m->topk_z : (double *)nullptr));
    RC(d->d2h(ids, m->topk_ids, sizeof(int) * (size_t)B * k));
    RC(d->d2h(vals, m->topk_vals, sizeof(float) * (size_t)B * k));
    if (want_z) RC(d->d2h(z, m->topk_z, sizeof(double) * (size_t)B));
    return RD_OK;
}

// TopKRow.Full: the whole logits row of the last step's row `row`, for the token where k entries were not enough. Valid until
// the next step.
extern "C" int rd_last_logits(rd_model *m, int row, float *logits) {
    if (!m || !logits || row < 0 || row >= m->last_B) {
        if (m) rd_set_error("rd_last_logits: row %d of a step of %d", row, m->last_B);
        return RD_ERR_ARG;
    }
    if (!m->last_logits_valid) {
        rd_set_error("rd_last_logits: the last step kept no logits");
        return RD_ERR_STATE;
    }
    return m->d->d2h(logits, m->logits + (size_t)row * m->desc.vocab, sizeof(float) * (size_t)m->desc.vocab);
}

extern "C" int rd_moe_replay(rd_model *m, int B, const int *idx, const float *wgt) {
    if (!m || !idx || !wgt || m->desc.n_experts == 0 || B < 1 || B > 32) {
        rd_set_error("rd_moe_replay: needs a MoE model, 1 <= B <= 32 and both arrays");
        return RD_ERR_ARG;
    }
    const int L = m->desc.n_layers, k = m->desc.top_k, nE = m->desc.n_experts;
    m->replay_idx.assign((size_t)L, std::vector<int>((size_t)B * k));
    m->replay_wgt.assign((size_t)L, std::vector<float>((size_t)B * k));
    m->replay_rank.assign((size_t)L, std::vector<signed char>((size_t)32 * nE, (signed char)-1));
    for (int b = 0; b < B; b++)
        for (int l = 0; l < L; l++)
            for (int j = 0; j < k; j++) {
                int e = idx[((size_t)b * L + l) * k + j];
                if (e < 0 || e >= nE) {
                    rd_set_error("rd_moe_replay: expert %d out of range at row %d layer %d", e, b, l);
                    m->replay_B = 0;
                    return RD_ERR_ARG;
                }
                m->replay_idx[(size_t)l][(size_t)b * k + j] = e;
                m->replay_wgt[(size_t)l][(size_t)b * k + j] = wgt[((size_t)b * L + l) * k + j];
                m->replay_rank[(size_t)l][(size_t)b * nE + e] = (signed char)j;
            }
    m->replay_B = B;
    return RD_OK;
}

extern "C" int rd_last_moe_indices(rd_model *m, int *idx) {
    if (!m || !idx || m->desc.n_experts == 0 || m->last_B == 0) return RD_ERR_ARG;
    rd_device *d = m->d;
    int k = m->desc.top_k, B = m->last_B;
    std::vector<int> all((size_t)m->desc.n_layers * 32 * k);
    RC(d->d2h(all.data(), m->moe_idx_all, sizeof(int) * all.size()));
    for (int b = 0; b < B; b++)
        for (int l = 0; l < m->desc.n_layers; l++)
            for (int j = 0; j < k; j++) idx[((size_t)b * m->desc.n_layers + l) * k + j] = all[((size_t)l * 32 + b) * k + j];
    return RD_OK;
}
