// device.cc — device open/close, code-object loading, memory helpers, weight upload and the GEMM launcher.
#include <algorithm>
#include "device.h"
#include <dlfcn.h>
#include <mutex>
#include <stdlib.h>
#include <string.h>

static thread_local char g_err[512] = "";

void rd_set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
}

bool rd_hip_ok(const HipApi *hip, hipError_t e, const char *what) {
    if (e == hipSuccess) return true;
    rd_set_error("%s: %s", what, hip ? hip->GetErrorString(e) : "hip not loaded");
    return false;
}

extern "C" const char *rd_last_error(void) { return g_err; }
extern "C" const char *rd_backend_name(void) { return "rocm"; }

int rd_device::use() { return rd_hip_ok(hip, hip->SetDevice(ordinal), "hipSetDevice") ? RD_OK : RD_ERR_HIP; }
int rd_device::alloc(void **p, size_t n) {
    if (use()) return RD_ERR_HIP;
    if (!rd_hip_ok(hip, hip->Malloc(p, n), "hipMalloc")) return RD_ERR_HIP;
    return RD_OK;
}
void rd_device::release(void *p) {
    if (p) (void)hip->Free(p);
}
int rd_device::h2d(void *dst, const void *src, size_t n) {
    if (use()) return RD_ERR_HIP;
    return rd_hip_ok(hip, hip->MemcpyAsync(dst, src, n, hipMemcpyHostToDevice, stream), "hipMemcpy H2D") ? RD_OK : RD_ERR_HIP;
}
int rd_device::d2h(void *dst, const void *src, size_t n) {
    if (!rd_hip_ok(hip, hip->MemcpyAsync(dst, src, n, hipMemcpyDeviceToHost, stream), "hipMemcpy D2H")) return RD_ERR_HIP;
    return sync();
}
int rd_device::sync() { return rd_hip_ok(hip, hip->StreamSynchronize(stream), "hipStreamSynchronize") ? RD_OK : RD_ERR_HIP; }

static bool read_file(const std::string &path, std::vector<char> &out) {
    FILE *f = fopen(path.c_str(), "rb");
    if (!f) return false;
    fseek(f, 0, SEEK_END);
    long n = ftell(f);
    fseek(f, 0, SEEK_SET);
    out.resize((size_t)n);
    bool ok = n > 0 && fread(out.data(), 1, (size_t)n, f) == (size_t)n;
    fclose(f);
    return ok;
}

// The code object sits beside this shared library unless ROCMDECODE_HSACO names it.
static std::string default_hsaco_path() {
    if (const char *e = getenv("ROCMDECODE_HSACO")) return e;
    Dl_info info;
    if (dladdr((void *)&rd_last_error, &info) && info.dli_fname) {
        std::string p = info.dli_fname;
        size_t s = p.find_last_of('/');
        return (s == std::string::npos ? std::string(".") : p.substr(0, s)) + "/rocmdecode_gfx950.hsaco";
    }
    return "rocmdecode_gfx950.hsaco";
}

struct KName {
    const char *name;
    hipFunction_t Kernels::*slot;
};
static const KName kNames[] = {
    {"rd_k_dequant_q4k", &Kernels::dequant_q4k},
    {"rd_k_quant_act", &Kernels::quant_act},
    {"rd_k_quant_act_row", &Kernels::quant_act_row},
    {"rd_k_swiglu_quant_row", &Kernels::swiglu_quant_row},
    {"rd_k_moe_gemv_w4a8r", &Kernels::moe_gemv_w4a8r},
    {"rd_k_moe_gemv_w4a8r_f32in", &Kernels::moe_gemv_w4a8r_f32in},
    {"rd_k_moe_gemv_w4a8r_gateup", &Kernels::moe_gemv_w4a8r_gateup},
    {"rd_k_moe_swiglu_quant_row", &Kernels::moe_swiglu_quant_row},
    {"rd_k_reduce_splits", &Kernels::reduce_splits},
    {"rd_k_add_rmsnorm_quant", &Kernels::add_rmsnorm_quant},
    {"rd_k_swiglu_quant", &Kernels::swiglu_quant},
    {"rd_k_unpack_act8", &Kernels::unpack_act8},
    {"rd_k_unpanel_a8", &Kernels::unpanel_a8},
    {"rd_k_retile_w8a8_8", &Kernels::retile_w8a8_8},
    {"rd_k_retile_w4a8_8", &Kernels::retile_w4a8_8},
    {"rd_k_gemm8_q4k_rows", &Kernels::gemm8_q4k_rows},
    {"rd_k_gemm8_q4k_rows_g2", &Kernels::gemm8_q4k_rows_g2},
    {"rd_k_gemm8_q5k_rows", &Kernels::gemm8_q5k_rows},
    {"rd_k_gemm8_q5k_rows_g2", &Kernels::gemm8_q5k_rows_g2},
    {"rd_k_gemm8_q6k_rows", &Kernels::gemm8_q6k_rows},
    {"rd_k_gemm8_q6k_rows_g2", &Kernels::gemm8_q6k_rows_g2},
    {"rd_k_gemm8_q4k_rows_gateup", &Kernels::gemm8_q4k_rows_gateup},
    {"rd_k_gemm8_q4k_rows_gateup_gelu", &Kernels::gemm8_q4k_rows_gateup_gelu},
    {"rd_k_gemm8_q4k_rows_qkv", &Kernels::gemm8_q4k_rows_qkv},
    {"rd_k_gemm8_q4k_rows_qkv_g2", &Kernels::gemm8_q4k_rows_qkv_g2},
    {"rd_k_gemm8_q4k_gateup", &Kernels::gemm8_q4k_gateup},
    {"rd_k_gemm8_q4k_gateup_gelu", &Kernels::gemm8_q4k_gateup_gelu},
    {"rd_k_gemm8_q4k_gateup_norm1", &Kernels::gemm8_q4k_gateup_norm1},
    {"rd_k_gemm8_q4k_gateup_gelu_norm1", &Kernels::gemm8_q4k_gateup_gelu_norm1},
    {"rd_k_add_one", &Kernels::add_one},
    {"rd_k_moe_gemv_w4a8", &Kernels::moe_gemv_w4a8},
    {"rd_k_moe_gemv_w4a8_gateup", &Kernels::moe_gemv_w4a8_gateup},
    {"rd_k_retile_w4a8_gv", &Kernels::retile_w4a8_gv},
    {"rd_k_retile_q4k8", &Kernels::retile_q4k8},
    {"rd_k_dequant_q5k", &Kernels::dequant_q5k},
    {"rd_k_retile_q5k", &Kernels::retile_q5k},
    {"rd_k_dequant_q6k", &Kernels::dequant_q6k},
    {"rd_k_retile_q6k", &Kernels::retile_q6k},
    {"rd_k_kv_store", &Kernels::kv_store},
    {"rd_k_kv_read", &Kernels::kv_read},
    {"rd_k_qkv_rope_store", &Kernels::qkv_rope_store},
    {"rd_k_rope_table", &Kernels::rope_table},
    {"rd_k_attn_partial", &Kernels::attn_partial},
    {"rd_k_attn_partial_wide", &Kernels::attn_partial_wide},
    {"rd_k_kv_store_i8", &Kernels::kv_store_i8},
    {"rd_k_qkv_rope_store_i8", &Kernels::qkv_rope_store_i8},
    {"rd_k_attn_partial_i8", &Kernels::attn_partial_i8},
    {"rd_k_attn_partial_deep", &Kernels::attn_partial_deep},
    {"rd_k_attn_partial_deep_i8", &Kernels::attn_partial_deep_i8},
    {"rd_k_attn_partial_rows", &Kernels::attn_partial_rows},
    {"rd_k_attn_partial_rows_i8", &Kernels::attn_partial_rows_i8},
    {"rd_k_attn_combine", &Kernels::attn_combine},
    {"rd_k_attn_combine_quant", &Kernels::attn_combine_quant},
    {"rd_k_rmsnorm", &Kernels::rmsnorm},
    {"rd_k_rope", &Kernels::rope},
    {"rd_k_argmax_rows", &Kernels::argmax_rows},
    {"rd_k_argmax_final", &Kernels::argmax_final},
    {"rd_k_matmul_f32", &Kernels::matmul_f32},
    {"rd_k_moe_route", &Kernels::moe_route},
    {"rd_k_topk_rows", &Kernels::topk_rows},
    {"rd_k_topk_hist", &Kernels::topk_hist},
    {"rd_k_topk_pick", &Kernels::topk_pick},
    {"rd_k_topk_finish", &Kernels::topk_finish},
    {"rd_k_moe_swiglu_quant", &Kernels::moe_swiglu_quant},
    {"rd_k_moe_fold", &Kernels::moe_fold},
    {"rd_k_embed_rows", &Kernels::embed_rows},
    {"rd_k_copy16", &Kernels::copy16},
    {"rd_k_fill_f16", &Kernels::fill_f16},
    {"rd_k_fill_f32", &Kernels::fill_f32},
    {"rd_k_issue_mfma_i8", &Kernels::issue_mfma_i8},
    {"rd_k_issue_mfma_f32", &Kernels::issue_mfma_f32},
    {"rd_k_issue_valu", &Kernels::issue_valu},
    {"rd_k_issue_all", &Kernels::issue_all},
};

static int open_common(int ordinal, const void *image, rd_device **out) {
    const char *why = nullptr;
    const HipApi *hip = hip_api(&why);
    if (!hip) {
        rd_set_error("%s", why);
        return RD_DECLINED; // no ROCm runtime on this machine: the backend declines, the caller stays on its CPU path
    }
    if (!rd_hip_ok(hip, hip->Init(0), "hipInit")) return RD_DECLINED;
    int n = 0;
    if (!rd_hip_ok(hip, hip->GetDeviceCount(&n), "hipGetDeviceCount") || n <= ordinal) {
        rd_set_error("no HIP device %d (count %d)", ordinal, n);
        return RD_DECLINED;
    }
    rd_device *d = new rd_device();
    d->hip = hip;
    d->ordinal = ordinal;
    if (!rd_hip_ok(hip, hip->SetDevice(ordinal), "hipSetDevice") || !rd_hip_ok(hip, hip->StreamCreate(&d->stream), "hipStreamCreate") ||
        !rd_hip_ok(hip, hip->ModuleLoadData(&d->module, image), "hipModuleLoadData(gfx950 code object)")) {
        delete d;
        return RD_ERR_HIP;
    }
    for (const KName &kn : kNames) {
        hipFunction_t f = nullptr;
        if (hip->ModuleGetFunction(&f, d->module, kn.name) != hipSuccess) {
            rd_set_error("code object lacks kernel %s", kn.name);
            (void)hip->ModuleUnload(d->module);
            (void)hip->StreamDestroy(d->stream);
            delete d;
            return RD_ERR_HIP;
        }
        d->k.*(kn.slot) = f;
    }
    static const char *kindName[7] = {"q4k", "w8a8", "w4a8", "w8a8r", "w4a8r", "q5k", "q6k"};
    static const int kwOf[3] = {2, 4, 8};
    for (int kind = 0; kind < 7; kind++)
        for (int i = 0; i < 6; i++) {
            char name[64];
            if (i < 3)
                snprintf(name, sizeof name, "rd_k_gemm8_%s_kw%d", kindName[kind], kwOf[i]);
            else
                snprintf(name, sizeof name, "rd_k_gemm8_%s_qkv_kw%d", kindName[kind], kwOf[i - 3]);
            if (hip->ModuleGetFunction(i < 3 ? &d->k.gemm8[kind][i] : &d->k.gemm8_qkv[kind][i - 3], d->module, name) != hipSuccess) {
                rd_set_error("code object lacks kernel %s", name);
                (void)hip->ModuleUnload(d->module);
                (void)hip->StreamDestroy(d->stream);
                delete d;
                return RD_ERR_HIP;
            }
        }
    for (int i = 0; i < 3; i++) {
        char name[64];
        snprintf(name, sizeof name, "rd_k_gemm8_q4k_qkv_norm1_kw%d", 2 << i);
        if (hip->ModuleGetFunction(&d->k.gemm8_q4k_qkv_norm1[i], d->module, name) != hipSuccess) {
            rd_set_error("code object lacks kernel %s", name);
            (void)hip->ModuleUnload(d->module);
            (void)hip->StreamDestroy(d->stream);
            delete d;
            return RD_ERR_HIP;
        }
    }
    topk_static_prepare_device(ordinal); // the allocation-free top-K's one-time set-up for this device, outside any capture
    *out = d;
    return RD_OK;
}

extern "C" int rd_device_open_image(int ordinal, const void *hsaco, size_t len, rd_device **out) {
    if (!hsaco || len == 0 || !out) {
        rd_set_error("rd_device_open_image: null image");
        return RD_ERR_ARG;
    }
    return open_common(ordinal, hsaco, out);
}

extern "C" int rd_device_open(int ordinal, rd_device **out) {
    if (!out) return RD_ERR_ARG;
    std::vector<char> img;
    std::string path = default_hsaco_path();
    if (!read_file(path, img)) {
        rd_set_error("cannot read gfx950 code object %s (build it with goinfer_amd/build.py)", path.c_str());
        return RD_ERR_STATE;
    }
    return open_common(ordinal, img.data(), out);
}

extern "C" void rd_device_close(rd_device *d) {
    if (!d) return;
    (void)d->use();
    (void)d->hip->StreamSynchronize(d->stream);
    for (void *p : d->owned) (void)d->hip->Free(p);
    (void)d->hip->ModuleUnload(d->module);
    (void)d->hip->StreamDestroy(d->stream);
    delete d;
}

extern "C" int rd_device_sync(rd_device *d) { return d ? d->sync() : RD_ERR_ARG; }

extern "C" int rd_device_mem_info(rd_device *d, size_t *free_b, size_t *total_b) {
    if (!d) return RD_ERR_ARG;
    HIPCHK(MemGetInfo(free_b, total_b));
    return RD_OK;
}

int topk_scratch_alloc(rd_device *d, int rows, int V, TopkScratch *s) {
    const size_t R = (size_t)rows, chunks = (size_t)(V + TOPK_CHUNK - 1) / TOPK_CHUNK;
    int rc = d->alloc((void **)&s->ghist, sizeof(int) * R * chunks * TOPK_BINS);
    if (!rc) rc = d->alloc((void **)&s->ccount, sizeof(int) * R);
    if (!rc) rc = d->alloc((void **)&s->gmax, sizeof(unsigned) * R * chunks);
    if (!rc) rc = d->alloc((void **)&s->cand_i, sizeof(int) * R * TOPK_CAP);
    if (!rc) rc = d->alloc((void **)&s->cand_v, sizeof(float) * R * TOPK_CAP);
    if (!rc) rc = d->alloc((void **)&s->invT, sizeof(float) * R);
    if (!rc) rc = d->alloc((void **)&s->zpart, sizeof(double) * R * chunks);
    if (rc) return rc;
    if (!rd_hip_ok(d->hip, d->hip->MemsetAsync(s->ccount, 0, sizeof(int) * R, d->stream), "memset")) return RD_ERR_HIP;
    return RD_OK;
}

int launch_topk(rd_device *d, const float *logits, int rows, int V, int k, float invT, bool rowsInvT, const TopkScratch &s, int *ids, float *vals,
                double *z) {
    const float *it = rowsInvT ? s.invT : nullptr;
    if (V < 2 * TOPK_CHUNK) // a narrow row: one block reads it a few times
        return d->launch(d->k.topk_rows, (unsigned)rows, 1, 1, 1024u, logits, V, k, invT, it, ids, vals, z);
    const unsigned chunks = (unsigned)((V + TOPK_CHUNK - 1) / TOPK_CHUNK);
    int rc = d->launch(d->k.topk_hist, chunks, (unsigned)rows, 1, 1024u, logits, V, s.ghist, s.gmax);
    if (!rc)
        rc = d->launch(d->k.topk_pick, chunks, (unsigned)rows, 1, 1024u, logits, V, k, invT, it, (const int *)s.ghist, (const unsigned *)s.gmax, s.cand_v,
                       s.cand_i, s.ccount, z ? s.zpart : (double *)nullptr);
    if (!rc)
        rc = d->launch(d->k.topk_finish, (unsigned)rows, 1, 1, 1024u, logits, V, k, (int)chunks, (const float *)s.cand_v,
                       (const int *)s.cand_i, s.ccount, (const double *)s.zpart, ids, vals, z);
    return rc;
}

AttnLaunch attn_partial_kernel(const rd_device *d, bool i8, bool grouped, size_t n_items) {
    if (grouped) return {i8 ? d->k.attn_partial_rows_i8 : d->k.attn_partial_rows, 1u};
    if (n_items <= (size_t)ATTN_DEEP_MAX_ITEMS && !getenv("ROCMDECODE_NO_DEEP_ATTN")) return {i8 ? d->k.attn_partial_deep_i8 : d->k.attn_partial_deep, 1u};
    if (i8) return {d->k.attn_partial_i8, 1u};
    if (n_items >= (size_t)ATTN_WIDE_MIN_ITEMS && n_items % ATTN_BLOCK_WAVES == 0 && !getenv("ROCMDECODE_NO_WIDE_ATTN"))
        return {d->k.attn_partial_wide, (unsigned)ATTN_BLOCK_WAVES};
    return {d->k.attn_partial, 1u};
}

const char *attn_partial_kernel_name(const rd_device *d, hipFunction_t f) {
    const Kernels &k = d->k;
    if (f == k.attn_partial_wide) return "rd_k_attn_partial_wide";
    if (f == k.attn_partial) return "rd_k_attn_partial";
    if (f == k.attn_partial_i8) return "rd_k_attn_partial_i8";
    if (f == k.attn_partial_deep) return "rd_k_attn_partial_deep";
    if (f == k.attn_partial_deep_i8) return "rd_k_attn_partial_deep_i8";
    if (f == k.attn_partial_rows) return "rd_k_attn_partial_rows";
    if (f == k.attn_partial_rows_i8) return "rd_k_attn_partial_rows_i8";
    return "?";
}

bool build_attn_worklist(const int *len, const int *slot, int G, int rows, int n_kv, std::vector<AttnItemH> &items, std::vector<int> &ranges,
                         int window) {
    auto first_block = [&](int r) { return window > 0 ? std::max(len[r] - window, 0) / 64 : 0; };
    static const bool no_groups = getenv("ROCMDECODE_NO_ATTN_GROUPS") != nullptr;
    const int maxGroup = (slot && !no_groups && G <= ATTN_TILE_ROWS) ? ATTN_TILE_ROWS / G : 1;
    struct Group {
        int row, n;
    };
    std::vector<Group> groups;
    for (int r = 0; r < rows;) {
        int n = 1;
        while (n < maxGroup && r + n < rows && slot[r + n] == slot[r] && len[r + n] == len[r] + n && (len[r + n] + 63) / 64 == (len[r] + 63) / 64 &&
               first_block(r + n) == first_block(r))
            n++;
        groups.push_back({r, n});
        r += n;
    }
    std::stable_sort(groups.begin(), groups.end(), [&](const Group &a, const Group &b) { return len[a.row] > len[b.row]; });
    items.clear();
    ranges.assign((size_t)rows * n_kv * ATTN_RANGE_INTS, 0);
    bool grouped = false;
    for (const Group &g : groups) {
        const int nb = (len[g.row] + 63) / 64, fb = first_block(g.row), chunk = attn_chunk_blocks(nb - fb);
        grouped = grouped || g.n > 1;
        for (int h = 0; h < n_kv; h++) {
            const int first = (int)items.size();
            for (int b0 = fb; b0 < nb; b0 += chunk) items.push_back({g.row, h | (g.n << 16), b0, std::min(nb, b0 + chunk)});
            for (int j = 0; j < g.n; j++) {
                int *rg = &ranges[((size_t)(g.row + j) * n_kv + h) * ATTN_RANGE_INTS];
                rg[0] = first, rg[1] = (int)items.size(), rg[2] = j;
            }
        }
    }
    if (!grouped)
        for (auto &it : items) it.kvh &= 0xffff;
    return grouped;
}

// ---- GEMM planning ----
// f16-MFMA kinds (Q5_K, Q6_K): split K so that about one block per CU is in flight; a split keeps at least two K-blocks.
// int8-MFMA kinds: enough waves to give every SIMD about two; K is cut inside the block first (KW waves per tile, their partial
// sums folded in LDS, nothing through memory) and across blocks only when eight waves per tile still leave SIMDs idle.
// The plan depends on the weight's shape only, never on the number of rows: a row is summed in the same order in any batch.
GemmPlan plan_gemm(int kind, int N, int nKB, int act_group) {
    GemmPlan p;
    if (is_gemm8_kind(kind)) {
        const int tiles = (N + 31) / 32;
        int want = (2048 + tiles - 1) / tiles; // waves per tile for two per SIMD
        want = std::min(want, std::max(1, nKB));
        p.kw = want >= 8 ? 8 : (want >= 4 ? 4 : 2);
        p.splits = 1;
        if (p.kw == 8) p.splits = std::max(1, std::min(want / 8, nKB / 8)); // every wave keeps at least one K-block
        if (const char *e = getenv("ROCMDECODE_GEMM8_KW")) p.kw = atoi(e) == 8 ? 8 : (atoi(e) == 2 ? 2 : 4);
        if (const char *e = getenv("ROCMDECODE_GEMM8_SPLITS")) p.splits = std::max(1, std::min(atoi(e), nKB));
        if (act_group == 0) p.splits = 1;
        p.kbPerSplit = (nKB + p.splits - 1) / p.splits;
        p.splits = (nKB + p.kbPerSplit - 1) / p.kbPerSplit;
        return p;
    }
    rd_set_error("plan_gemm: unknown weight kind %d", kind);
    p.splits = 1, p.kbPerSplit = nKB, p.kw = 2;
    return p;
}

size_t panel_bytes_for(const DevWeight &w) { return a8_bytes(w.K); }
int panel_kind_for(const DevWeight &) { return PANEL_A8; }
int act_group_for(const DevWeight &w) { return w.kind == WKIND_GROUP ? (w.parts.empty() ? 32 : w.parts[0].act_group) : w.act_group; }
int launch_quant_act(rd_device *d, const float *x, int M, int K, int kind, int act_group, void *Xp) {
    if (act_group == 0) return d->launch(d->k.quant_act_row, (unsigned)M, 1, 1, 1024, x, Xp, K, kind);
    return d->launch(d->k.quant_act, (unsigned)((K + 255) / 256), (unsigned)M, 1, 256, x, Xp, K, kind);
}

int upload_q4k(rd_device *d, const void *blocks, int N, int K, DevWeight *w) {
    if (N <= 0 || K <= 0 || K % 256 || N % 32) {
        rd_set_error("q4k upload: N=%d must be a multiple of 32 and K=%d of 256", N, K);
        return RD_DECLINED;
    }
    size_t bytes = (size_t)N * (K / 256) * 144;
    DevBuf raw(d);
    int rc = raw.alloc(bytes);
    if (rc) return rc;
    if ((rc = d->alloc(&w->tiled, bytes))) return rc;
    if ((rc = d->h2d(raw.p, blocks, bytes))) return rc;
    int nSB = K / 256;
    if ((rc = d->launch(d->k.retile_q4k8, N / 32, nSB, 1, 320, (const void *)raw.p, w->tiled, N, nSB))) return rc;
    if ((rc = d->sync())) return rc;
    w->kind = 0, w->N = N, w->K = K;
    return RD_OK;
}

// Q5_K: 176 B super-blocks re-tiled to 5632 B per (32 rows, super-block), the file's own bits. Q6_K: 210 B super-blocks re-tiled
// to 7168 B per (32 rows, super-block): the int8 scales and d per lane half, nibbles, high bit pairs; 7 bits per weight against 6.5625 raw.
int upload_q5k(rd_device *d, const void *blocks, int N, int K, DevWeight *w) {
    if (N <= 0 || K <= 0 || K % 256 || N % 32) {
        rd_set_error("q5k upload: N=%d must be a multiple of 32 and K=%d of 256", N, K);
        return RD_DECLINED;
    }
    int nSB = K / 256;
    size_t bytes = (size_t)N * nSB * 176;
    DevBuf raw(d);
    int rc = raw.alloc(bytes);
    if (rc) return rc;
    if ((rc = d->alloc(&w->tiled, (size_t)(N / 32) * nSB * 5632))) return rc;
    if ((rc = d->h2d(raw.p, blocks, bytes))) return rc;
    if ((rc = d->launch(d->k.retile_q5k, N / 32, nSB, 1, 384, (const void *)raw.p, w->tiled, N, nSB))) return rc;
    if ((rc = d->sync())) return rc;
    w->kind = 3, w->N = N, w->K = K;
    return RD_OK;
}

int upload_q6k(rd_device *d, const void *blocks, int N, int K, DevWeight *w) {
    if (N <= 0 || K <= 0 || K % 256 || N % 32) {
        rd_set_error("q6k upload: N=%d must be a multiple of 32 and K=%d of 256", N, K);
        return RD_DECLINED;
    }
    int nSB = K / 256;
    size_t bytes = (size_t)N * nSB * 210;
    DevBuf raw(d);
    int rc = raw.alloc(bytes);
    if (rc) return rc;
    if ((rc = d->alloc(&w->tiled, (size_t)(N / 32) * nSB * 7168))) return rc;
    if ((rc = d->h2d(raw.p, blocks, bytes))) return rc;
    if ((rc = d->launch(d->k.retile_q6k, N / 32, nSB, 1, 448, (const void *)raw.p, w->tiled, N, nSB))) return rc;
    if ((rc = d->sync())) return rc;
    w->kind = 4, w->N = N, w->K = K;
    return RD_OK;
}

static bool act_group_ok(int g) {
    if (g == 0 || g == 32) return true;
    rd_set_error("rocm resident declines: activation quantization group %d (32 = per group of 32, 0 = one scale per row)", g);
    return false;
}

int upload_w8a8(rd_device *d, const int8_t *q, const float *row_scale, int N, int K, DevWeight *w, int act_group) {
    if (N <= 0 || K <= 0 || K % 32 || N % 32) {
        rd_set_error("w8a8 upload: N=%d and K=%d must be multiples of 32", N, K);
        return RD_DECLINED;
    }
    if (!act_group_ok(act_group)) return RD_DECLINED;
    size_t bytes = (size_t)N * K;
    const int nKB = (K + 255) / 256;
    DevBuf raw(d);
    int rc = raw.alloc(bytes);
    if (rc) return rc;
    if ((rc = d->alloc(&w->tiled, (size_t)(N / 32) * nKB * 8192))) return rc;
    if ((rc = d->alloc(&w->scales, sizeof(float) * (size_t)N))) return rc;
    if ((rc = d->h2d(raw.p, q, bytes))) return rc;
    if ((rc = d->h2d(w->scales, row_scale, sizeof(float) * (size_t)N))) return rc;
    if ((rc = d->launch(d->k.retile_w8a8_8, N / 32, nKB, 1, 512, (const void *)raw.p, w->tiled, N, K))) return rc;
    if ((rc = d->sync())) return rc;
    w->kind = 1, w->N = N, w->K = K, w->act_group = act_group;
    return RD_OK;
}

int upload_w4a8(rd_device *d, const uint8_t *nib, const uint16_t *s16, int N, int K, DevWeight *w, bool expert, int act_group) {
    if (N <= 0 || K <= 0 || K % 32 || N % 32) {
        rd_set_error("w4a8 upload: N=%d and K=%d must be multiples of 32", N, K);
        return RD_DECLINED;
    }
    if (!act_group_ok(act_group)) return RD_DECLINED;
    size_t nb = (size_t)N * K / 2, sb = (size_t)N * (K / 32) * 2;
    const int nKB = (K + 255) / 256;
    DevBuf raw(d), rs(d);
    int rc;
    if ((rc = raw.alloc(nb)) || (rc = rs.alloc(sb))) return rc;
    if ((rc = d->alloc(&w->tiled, (size_t)(N / 32) * nKB * 4608))) return rc;
    if ((rc = d->h2d(raw.p, nib, nb)) || (rc = d->h2d(rs.p, s16, sb))) return rc;
    // an expert's weights take the tile order of the vector-ALU kernels (moe.h), a dense projection's that of the MFMA kernels
    if ((rc = d->launch(expert ? d->k.retile_w4a8_gv : d->k.retile_w4a8_8, N / 32, nKB, 1, 320, (const void *)raw.p, (const void *)rs.p, w->tiled, N, K))) return rc;
    if ((rc = d->sync())) return rc;
    w->kind = 2, w->N = N, w->K = K, w->act_group = act_group;
    return RD_OK;
}

void free_weight(rd_device *d, DevWeight *w) {
    for (auto &p : w->parts) free_weight(d, &p);
    d->release(w->tiled);
    d->release(w->scales);
    *w = DevWeight();
}

bool rows_gemm_enabled() { return !getenv("ROCMDECODE_NO_ROWS_GEMM"); }

int launch_gemm(rd_device *d, const DevWeight &w, const void *Xp, float *P, int M, GemmPlan *plan_out, int ldP, int splits, int kw, float *resid,
                size_t xpStride, size_t pStride) {
    if (M < 1 || M > GEMM_WIDE_ROWS) { // rows past 32 are further M-tiles, grid.z of the launch
        rd_set_error("gemm: M=%d outside 1..32", M);
        return RD_ERR_ARG;
    }
    int nKB = kblocks_for(w);
    GemmPlan p = plan_gemm(w.kind, w.N, nKB, w.act_group);
    if (resid) splits = 1;
    if (w.act_group == 0 && is_gemm8_kind(w.kind) && splits > 1) {
        rd_set_error("gemm: a weight with per-row activation scales runs in one split (asked for %d)", splits);
        return RD_ERR_STATE;
    }
    if (splits > 0) p.kbPerSplit = (nKB + splits - 1) / splits, p.splits = splits;
    if (kw > 0) p.kw = kw;
    if (plan_out) *plan_out = p;
    if (ldP <= 0) ldP = w.N;
    if (is_gemm8_kind(w.kind)) {
        const int tiles = w.N / 32, tpb = p.kw == 2 ? 2 : 1;
        // more than 32 rows of Q4_K: four M-tiles share each decoded weight tile (the same sums, row for row)
        const int lane8 = gemm8_lane(w);
        if ((lane8 == 0 || lane8 == 5 || lane8 == 6) && M >= ROWS_GEMM_MIN_ROWS && rows_gemm_enabled()) { // Q4_K, Q5_K, Q6_K
            const unsigned gz = (unsigned)((M + 127) / 128);
            const bool two = rows_gemm_two_groups((size_t)tiles * p.splits * gz);
            hipFunction_t f = lane8 == 0 ? (two ? d->k.gemm8_q4k_rows_g2 : d->k.gemm8_q4k_rows)
                                         : (lane8 == 5 ? (two ? d->k.gemm8_q5k_rows_g2 : d->k.gemm8_q5k_rows) : (two ? d->k.gemm8_q6k_rows_g2 : d->k.gemm8_q6k_rows));
            return d->launch(f, (unsigned)tiles, (unsigned)p.splits, gz, two ? 512 : 256, (const void *)w.tiled, Xp, P, w.N, nKB, p.kbPerSplit, p.kw, M, ldP, resid,
                             xpStride, pStride);
        }
        hipFunction_t f = d->k.gemm8[gemm8_lane(w)][p.kw == 8 ? 2 : (p.kw == 4 ? 1 : 0)];
        return d->launch(f, (unsigned)((tiles + tpb - 1) / tpb), (unsigned)p.splits, (unsigned)((M + 31) / 32), (unsigned)(64 * p.kw * tpb), (const void *)w.tiled,
                         (const void *)w.scales, Xp, P, w.N, nKB, p.kbPerSplit, M, ldP, resid, xpStride, pStride);
    }
    rd_set_error("gemm: unknown weight kind %d", w.kind);
    return RD_ERR_STATE;
}

int launch_gemm_wide(rd_device *d, const DevWeight &w, const void *Xp, size_t xpStride, float *P, size_t pStride, int M, GemmPlan *plan_out, int ldP,
                     int splits, int kw) {
    if (M < 1 || M > GEMM_WIDE_ROWS) {
        rd_set_error("wide gemm: M=%d outside 1..%d", M, GEMM_WIDE_ROWS);
        return RD_ERR_ARG;
    }
    return launch_gemm(d, w, Xp, P, M, plan_out, ldP, splits, kw, nullptr, xpStride, pStride); // all M-tiles in one launch
}
