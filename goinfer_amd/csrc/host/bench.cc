// bench.cc — measurement entry points: HIP-event timing on the stream the kernels are launched on, with every input
// already resident in HBM when the timed region starts.
#include "model.h"
#include <algorithm>
#include <chrono>
#include <memory>
#include <numeric>
#include <string.h>
#include <string>

#define RC(x)                \
    do {                     \
        int rd_rc_macro_ = (x); \
        if (rd_rc_macro_) return rd_rc_macro_; \
    } while (0)

// Greedy decode chain entirely on the device: ids0 are the first tokens; every step embeds the previous step's argmax
// (rd_model_upload_embedding), runs the ragged batched step and picks the next ids. ms_out[steps] are per-step
// milliseconds; ids_out (optional) [steps][B] are the tokens picked.
extern "C" int rd_bench_steps(rd_model *m, int B, const int *slot, const int *pos0, const int *ids0, int warmup, int steps, float *ms_out,
                              int *ids_out) {
    if (!m || !slot || !pos0 || !ids0 || !ms_out || steps <= 0 || warmup < 0 || B < 1 || B > m->max_rows) return RD_ERR_ARG;
    rd_device *d = m->d;
    RC(d->h2d(m->ids, ids0, sizeof(int) * (size_t)B));
    RC(d->sync());
    // One event per step boundary; nothing is waited for until the last step is enqueued, so the host runs ahead of the
    // GPU as a serving loop chaining greedy steps on the device would (ids_out asks for a read-back per step instead).
    const int total = warmup + steps;
    std::vector<hipEvent_t> ev((size_t)total + 1);
    for (auto &e : ev) HIPCHK(EventCreate(&e));
    std::vector<int> pos((size_t)B);
    int rc = RD_OK;
    (void)d->hip->EventRecord(ev[0], d->stream);
    for (int i = 0; i < total && !rc; i++) {
        for (int b = 0; b < B; b++) pos[(size_t)b] = pos0[b] + i;
        rc = model_step(m, B, slot, pos.data(), nullptr, nullptr, RD_WANT_ARGMAX, nullptr, nullptr);
        (void)d->hip->EventRecord(ev[(size_t)i + 1], d->stream);
        if (i >= warmup && ids_out && !rc) rc = d->d2h(ids_out + (size_t)(i - warmup) * B, m->ids, sizeof(int) * (size_t)B);
    }
    if (!rc) rc = d->sync();
    for (int i = warmup; i < total; i++) {
        float ms = 0.f;
        if (!rc) (void)d->hip->EventElapsedTime(&ms, ev[(size_t)i], ev[(size_t)i + 1]);
        ms_out[i - warmup] = ms;
    }
    for (auto &e : ev) (void)d->hip->EventDestroy(e);
    return rc;
}

// The host's own cost of a step: `steps` chained greedy steps are enqueued without waiting for the GPU and the wall clock of the
// enqueue loop alone is taken (the stream is drained before and after). *host_us = microseconds of host time per step. With more
// steps than the staging ring has slots (rd_model::STAGE_SLOTS) the loop waits for the GPU and measures that instead.
extern "C" int rd_bench_enqueue(rd_model *m, int B, const int *slot, const int *pos0, const int *ids0, int steps, double *host_us) {
    if (!m || !slot || !pos0 || !ids0 || !host_us || steps <= 0 || B < 1 || B > m->max_rows) return RD_ERR_ARG;
    rd_device *d = m->d;
    RC(d->h2d(m->ids, ids0, sizeof(int) * (size_t)B));
    std::vector<int> pos((size_t)B);
    int rc = RD_OK;
    for (int i = 0; i < 3 && !rc; i++) { // settle: the third step with one key runs from the graph when graphs are on
        for (int b = 0; b < B; b++) pos[(size_t)b] = pos0[b] + i;
        rc = model_step(m, B, slot, pos.data(), nullptr, nullptr, RD_WANT_ARGMAX, nullptr, nullptr);
    }
    RC(d->sync());
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 3; i < 3 + steps && !rc; i++) {
        for (int b = 0; b < B; b++) pos[(size_t)b] = pos0[b] + i;
        rc = model_step(m, B, slot, pos.data(), nullptr, nullptr, RD_WANT_ARGMAX, nullptr, nullptr);
    }
    const auto t1 = std::chrono::steady_clock::now();
    const int rc2 = d->sync();
    *host_us = std::chrono::duration<double, std::micro>(t1 - t0).count() / steps;
    return rc ? rc : rc2;
}

// One step with an event pair around every kernel class: class_ms[KC_COUNT] total milliseconds, class_n[KC_COUNT] launches.
extern "C" int rd_bench_profile(rd_model *m, int B, const int *slot, const int *pos, const int *ids0, float *class_ms, int *class_n) {
    if (!m || !slot || !pos || !ids0 || !class_ms || !class_n) return RD_ERR_ARG;
    rd_device *d = m->d;
    RC(d->h2d(m->ids, ids0, sizeof(int) * (size_t)B));
    RC(d->sync());
    m->timer.on = true;
    int rc = model_step(m, B, slot, pos, nullptr, nullptr, RD_WANT_ARGMAX, nullptr, nullptr);
    m->timer.on = false;
    int rc2 = d->sync();
    memset(class_ms, 0, sizeof(float) * KC_COUNT);
    memset(class_n, 0, sizeof(int) * KC_COUNT);
    for (size_t i = 0; i < m->timer.cls.size(); i++) {
        float ms = 0.f;
        if (!rc && !rc2) (void)d->hip->EventElapsedTime(&ms, m->timer.ev[2 * i], m->timer.ev[2 * i + 1]);
        class_ms[m->timer.cls[i]] += ms;
        class_n[m->timer.cls[i]]++;
    }
    for (hipEvent_t e : m->timer.ev) (void)d->hip->EventDestroy(e);
    m->timer.ev.clear(), m->timer.cls.clear();
    return rc ? rc : rc2;
}

// The attention kernel's average launch duration without an event pair around every launch: one step as in rd_bench_profile
// (which leaves its work list, q rows and KV on the device), then the kernel of every layer launched back to back `reps` times
// between ONE pair of events on the launch stream. *ms_per_launch = elapsed / (layers * reps); *launches = layers * reps.
extern "C" int rd_bench_attn_chain(rd_model *m, int B, const int *slot, const int *pos, const int *ids0, int reps, float *ms_per_launch, int *launches) {
    if (!m || !slot || !pos || !ids0 || !ms_per_launch || !launches || reps < 1) return RD_ERR_ARG;
    rd_device *d = m->d;
    RC(d->h2d(m->ids, ids0, sizeof(int) * (size_t)B));
    RC(model_step(m, B, slot, pos, nullptr, nullptr, RD_WANT_ARGMAX, nullptr, nullptr));
    RC(d->sync());
    hipEvent_t a, b2;
    (void)d->hip->EventCreate(&a), (void)d->hip->EventCreate(&b2);
    int rc = RD_OK;
    (void)d->hip->EventRecord(a, d->stream);
    for (int r = 0; r < reps && !rc; r++)
        for (auto &l : m->layers)
            if ((rc = launch_attn_partial(m, l))) break;
    (void)d->hip->EventRecord(b2, d->stream);
    int rc2 = d->sync();
    float ms = 0.f;
    if (!rc && !rc2) (void)d->hip->EventElapsedTime(&ms, a, b2);
    (void)d->hip->EventDestroy(a), (void)d->hip->EventDestroy(b2);
    *launches = reps * (int)m->layers.size();
    *ms_per_launch = ms / (float)*launches;
    return rc ? rc : rc2;
}

// The attention kernel the model's last step launched for its whole-context work list (names the kernel a roofline is for).
extern "C" const char *rd_bench_attn_kernel_name(rd_model *m) {
    if (!m || !m->last_items[0]) return "";
    return attn_partial_kernel_name(m->d, attn_partial_kernel(m->d, m->kv_type == RD_KV_I8, m->last_grouped[0], m->last_items[0]).f);
}

// The attention kernel's cost where it runs, inside the step: `reps` pairs of steps at the same positions, one whole and one with the
// attention launches left out, each between its own pair of events; *ms_per_launch = (mean whole - mean without) / layers. Unlike
// the back-to-back chain above, the kernel here starts as it does in service: behind the q|k|v projection, with the work list,
// the tables and q not yet in any L2.
extern "C" int rd_bench_attn_in_step(rd_model *m, int B, const int *slot, const int *pos, const int *ids0, int reps, float *ms_per_launch, float *ms_step) {
    if (!m || !slot || !pos || !ids0 || !ms_per_launch || reps < 1) return RD_ERR_ARG;
    rd_device *d = m->d;
    RC(d->h2d(m->ids, ids0, sizeof(int) * (size_t)B));
    RC(model_step(m, B, slot, pos, nullptr, nullptr, RD_WANT_ARGMAX, nullptr, nullptr)); // settle: the positions exist from here on
    RC(d->sync());
    std::vector<hipEvent_t> ev((size_t)reps * 4);
    for (auto &e : ev) HIPCHK(EventCreate(&e));
    int rc = RD_OK;
    for (int r = 0; r < reps && !rc; r++)
        for (int skip = 0; skip < 2 && !rc; skip++) {
            m->bench_skip_attn = skip != 0;
            (void)d->hip->EventRecord(ev[(size_t)r * 4 + 2 * skip], d->stream);
            rc = model_step(m, B, slot, pos, nullptr, nullptr, RD_WANT_ARGMAX, nullptr, nullptr);
            (void)d->hip->EventRecord(ev[(size_t)r * 4 + 2 * skip + 1], d->stream);
        }
    m->bench_skip_attn = false;
    const int rc2 = d->sync();
    // the median over the pairs of (step - step without attention): a pair that caught a clock change or another process's burst
    // does not move it
    std::vector<double> diff((size_t)reps), whole((size_t)reps);
    for (int r = 0; r < reps; r++) {
        float a = 0.f, b = 0.f;
        if (!rc && !rc2) {
            (void)d->hip->EventElapsedTime(&a, ev[(size_t)r * 4], ev[(size_t)r * 4 + 1]);
            (void)d->hip->EventElapsedTime(&b, ev[(size_t)r * 4 + 2], ev[(size_t)r * 4 + 3]);
        }
        diff[(size_t)r] = (double)a - (double)b, whole[(size_t)r] = a;
    }
    for (auto &e : ev) (void)d->hip->EventDestroy(e);
    auto median = [](std::vector<double> v) {
        std::sort(v.begin(), v.end());
        const size_t n = v.size();
        return n % 2 ? v[n / 2] : 0.5 * (v[n / 2 - 1] + v[n / 2]);
    };
    *ms_per_launch = (float)(median(diff) / (double)m->layers.size());
    if (ms_step) *ms_step = (float)median(whole);
    return rc ? rc : rc2;
}

// A prompt pass with every input on the device: rows 0..n-1 of `slot` from token ids through the embedding table, in the passes
// rd_prefill_last makes (all rows but the last build only their K/V, as wide as the step goes; the last is a one-row step with
// the head). ms_total: the whole prompt, HIP events on the launch stream. profile != 0: an event pair around every kernel class
// as in rd_bench_profile (the pairs stretch the run; take ms_total from a call without them).
extern "C" int rd_bench_prefill(rd_model *m, int slot, int n, const int *ids, int profile, float *ms_total, float *class_ms, int *class_n) {
    if (!m || !ids || !ms_total || n < 1 || (profile && (!class_ms || !class_n))) return RD_ERR_ARG;
    if (!m->embed_q || !m->tables || slot < 0 || slot >= m->slots || n > m->ctx_cap) {
        rd_set_error("rd_bench_prefill: needs the embedding table, a configured KV pool, a slot in range and n within the context cap");
        return RD_ERR_STATE;
    }
    rd_device *d = m->d;
    RC(rd_kv_reset(m, slot));
    int *ids_dev = nullptr;
    RC(d->alloc((void **)&ids_dev, sizeof(int) * (size_t)n));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    int rc = d->h2d(ids_dev, ids, sizeof(int) * (size_t)n);
    if (!rc) rc = d->sync();
    if (!rc && (d->hip->EventCreate(&e0) != hipSuccess || d->hip->EventCreate(&e1) != hipSuccess)) rc = RD_ERR_HIP;
    const int pass = m->max_rows;
    std::vector<int> rslot((size_t)pass, slot), rpos((size_t)pass);
    m->timer.on = profile != 0;
    if (!rc) (void)d->hip->EventRecord(e0, d->stream);
    auto run = [&](int r0, int rows, int want) {
        for (int j = 0; j < rows; j++) rpos[(size_t)j] = r0 + j;
        if (!rd_hip_ok(d->hip, d->hip->MemcpyAsync(m->ids, ids_dev + r0, sizeof(int) * (size_t)rows, hipMemcpyDeviceToDevice, d->stream), "hipMemcpy D2D"))
            return (int)RD_ERR_HIP;
        return model_step(m, rows, rslot.data(), rpos.data(), nullptr, nullptr, want, nullptr, nullptr, true);
    };
    for (int r0 = 0; r0 < n - 1 && !rc; r0 += pass) rc = run(r0, std::min(pass, n - 1 - r0), 0);
    if (!rc) rc = run(n - 1, 1, RD_WANT_ARGMAX);
    m->timer.on = false;
    if (!rc) (void)d->hip->EventRecord(e1, d->stream);
    int rc2 = d->sync();
    *ms_total = 0.f;
    if (!rc && !rc2) (void)d->hip->EventElapsedTime(ms_total, e0, e1);
    if (profile) {
        memset(class_ms, 0, sizeof(float) * KC_COUNT);
        memset(class_n, 0, sizeof(int) * KC_COUNT);
        for (size_t i = 0; i < m->timer.cls.size(); i++) {
            float ms = 0.f;
            if (!rc && !rc2) (void)d->hip->EventElapsedTime(&ms, m->timer.ev[2 * i], m->timer.ev[2 * i + 1]);
            class_ms[m->timer.cls[i]] += ms;
            class_n[m->timer.cls[i]]++;
        }
    }
    for (hipEvent_t e : m->timer.ev) (void)d->hip->EventDestroy(e);
    m->timer.ev.clear(), m->timer.cls.clear();
    if (e0) (void)d->hip->EventDestroy(e0);
    if (e1) (void)d->hip->EventDestroy(e1);
    d->release(ids_dev);
    return rc ? rc : rc2;
}

extern "C" int rd_bench_class_count(void) { return KC_COUNT; }
extern "C" const char *rd_bench_class_name(int c) {
    static const char *names[KC_COUNT] = {"gemm_qkv", "rope_kvstore", "attn_partial", "attn_combine", "gemm_o", "add_rmsnorm_quant", "gemm_gateup",
                                          "swiglu_quant", "gemm_down", "gemm_head", "argmax", "moe_router", "moe_gemm_gateup", "moe_gemm_down", "moe_glue"};
    return c >= 0 && c < KC_COUNT ? names[c] : "";
}

// Kernel micro-benchmarks over resident synthetic operands.
//   "gemm_q4k", "gemm_q5k", "gemm_q6k"  args {N, K, M, copies}: dst = a . W^T on `copies` distinct weight copies used round-robin (so the 256 MB
//               Infinity Cache cannot hold the weights between launches); operands are random bytes with sane f16 scales.
//   "gateup"    args {I, K, M, copies}: the fused gate|up projection + SwiGLU + quantization kernel.
//   "copy"      args {bytes}: a plain 16-byte-per-lane copy kernel over `bytes` (a multiple of 16), the yardstick for
//               scaling hardware traffic counters and for the practical HBM rate.
//   "issue"     args {mode, waves, iterations[, compute units = 256]}: the issue-rate probes (rd_k_issue_*: mode 0 int8 MFMAs, 1 f32 MFMAs, 2 the fold's
//               vector instructions, 3 all of them) with `waves` (1..2) waves on every SIMD; no memory traffic in the loop.
// ms_out[iters]: per-launch milliseconds (HIP events on the launch stream).
extern "C" int rd_bench_kernel(rd_device *d, const char *name, const int64_t *args, int n_args, int warmup, int iters, float *ms_out) {
    if (!d || !name || !args || iters <= 0 || !ms_out) return RD_ERR_ARG;
    std::string nm(name);
    const bool isGemm = nm == "gemm_q4k" || nm == "gemm_q5k" || nm == "gemm_q6k";
    if (isGemm && n_args >= 4 && (args[0] % 32 || args[1] % 256 || args[0] <= 0 || args[1] <= 0 || args[2] < 1 || args[2] > GEMM_WIDE_ROWS)) {
        rd_set_error("%s bench: bad shape", name);
        return RD_ERR_ARG;
    }
    if (nm == "gateup" && n_args >= 4 && (args[0] <= 0 || args[0] % 64 || args[1] <= 0 || args[1] % 256 || args[2] < 1 || args[2] > 64)) {
        rd_set_error("gateup bench: bad shape");
        return RD_ERR_ARG;
    }
    if (nm == "copy" && n_args >= 1 && (args[0] <= 0 || args[0] % 16)) {
        rd_set_error("copy bench: bytes must be a positive multiple of 16");
        return RD_ERR_ARG;
    }
    std::vector<hipEvent_t> ev((size_t)iters * 2);
    for (auto &e : ev) HIPCHK(EventCreate(&e));
    int rc = RD_OK;
    if (isGemm && n_args >= 4) {
        int N = (int)args[0], K = (int)args[1], M = (int)args[2], copies = (int)std::max<int64_t>(1, args[3]);
        const int kind = nm == "gemm_q4k" ? 0 : (nm == "gemm_q5k" ? 3 : 4), bb = kind == 0 ? 144 : (kind == 3 ? 176 : 210);
        size_t bytes = (size_t)N * (K / 256) * bb;
        std::vector<uint8_t> raw(bytes);
        uint64_t s = 88172645463325252ULL;
        for (size_t i = 0; i < bytes; i++) {
            s ^= s << 13, s ^= s >> 7, s ^= s << 17;
            raw[i] = (uint8_t)s;
        }
        for (size_t b = 0; b < bytes / bb; b++) { // small finite f16 super-scales
            uint8_t *blk = raw.data() + b * bb;
            if (kind == 4)
                blk[209] = 0x10 | (blk[209] & 3);
            else
                blk[1] = 0x10 | (blk[1] & 3), blk[3] = 0x10 | (blk[3] & 3);
        }
        std::vector<DevWeight> ws((size_t)copies);
        for (auto &w : ws)
            if (!rc) rc = kind == 0 ? upload_q4k(d, raw.data(), N, K, &w) : (kind == 3 ? upload_q5k(d, raw.data(), N, K, &w) : upload_q6k(d, raw.data(), N, K, &w));
        DevBuf Xp(d), P(d), X(d);
        const int pkind = PANEL_A8;
        size_t pb = a8_bytes(K);
        const int tiles = (M + 31) / 32; // rows beyond 32 are further M-tiles, each with its own panels and partial sums
        if (!rc) rc = Xp.alloc(pb * tiles);
        int nKB = K / kblock_of(kind);
        GemmPlan plan = plan_gemm(kind, N, nKB);
        const size_t pStride = (size_t)plan.splits * 32 * N;
        if (!rc) rc = P.alloc(sizeof(float) * pStride * tiles);
        if (!rc) rc = X.alloc(sizeof(float) * (size_t)32 * K);
        if (!rc) rc = d->launch(d->k.fill_f32, 256, 1, 1, 256, X.as<float>(), (size_t)32 * K, 7u); // the same 32 rows for every M-tile
        for (int t = 0; t < tiles && !rc; t++)
            rc = d->launch(d->k.quant_act, (unsigned)((K + 255) / 256), 32u, 1, 256, (const float *)X.p, (uint8_t *)Xp.p + (size_t)t * pb, K, pkind);
        if (!rc) rc = d->sync();
        for (int i = 0; i < warmup + iters && !rc; i++) {
            const DevWeight &w = ws[(size_t)i % ws.size()];
            if (i >= warmup) (void)d->hip->EventRecord(ev[2 * (size_t)(i - warmup)], d->stream);
            rc = launch_gemm_wide(d, w, Xp.p, pb, P.as<float>(), pStride, M, nullptr); // M-tiles of 32 rows
            if (i >= warmup) (void)d->hip->EventRecord(ev[2 * (size_t)(i - warmup) + 1], d->stream);
        }
        if (!rc) rc = d->sync();
        for (auto &w : ws) free_weight(d, &w);
    } else if (nm == "gateup" && n_args >= 4) {
        // args {I, K, M, copies}: the fused gate|up + SwiGLU + quantization kernel on `copies` weight sets used round-robin
        int I = (int)args[0], K = (int)args[1], M = (int)args[2], copies = (int)std::max<int64_t>(1, args[3]);
        size_t bytes = (size_t)2 * I * (K / 256) * 144;
        std::vector<uint8_t> raw(bytes);
        uint64_t s = 88172645463325252ULL;
        for (size_t i = 0; i < bytes; i++) {
            s ^= s << 13, s ^= s >> 7, s ^= s << 17;
            raw[i] = (uint8_t)s;
        }
        for (size_t b = 0; b < bytes / 144; b++) raw[b * 144 + 1] = 0x10 | (raw[b * 144 + 1] & 3), raw[b * 144 + 3] = 0x10 | (raw[b * 144 + 3] & 3);
        std::vector<DevWeight> ws((size_t)copies);
        for (auto &w : ws)
            if (!rc) rc = upload_q4k(d, raw.data(), 2 * I, K, &w);
        DevBuf Xp(d), Xo(d), X(d);
        if (!rc) rc = Xp.alloc(a8_bytes(K));
        if (!rc) rc = Xo.alloc(a8_bytes(I));
        if (!rc) rc = X.alloc(sizeof(float) * (size_t)32 * K);
        if (!rc) rc = d->launch(d->k.fill_f32, 256, 1, 1, 256, X.as<float>(), (size_t)32 * K, 7u);
        if (!rc) rc = d->launch(d->k.quant_act, (unsigned)((K + 255) / 256), 32u, 1, 256, (const float *)X.p, (uint8_t *)Xp.p, K, (int)PANEL_A8);
        if (!rc) rc = d->sync();
        for (int i = 0; i < warmup + iters && !rc; i++) {
            const DevWeight &w = ws[(size_t)i % ws.size()];
            if (i >= warmup) (void)d->hip->EventRecord(ev[2 * (size_t)(i - warmup)], d->stream);
            for (int m0 = 0; m0 < M && !rc; m0 += 32)
                rc = d->launch(d->k.gemm8_q4k_gateup, (unsigned)(I / 32), 1, 1, GATEUP_THREADS, (const void *)w.tiled, (const void *)Xp.p, Xo.as<uint8_t>(),
                               (int)PANEL_A8, I, K / 256, std::min(32, M - m0), (size_t)0, (size_t)0);
            if (i >= warmup) (void)d->hip->EventRecord(ev[2 * (size_t)(i - warmup) + 1], d->stream);
        }
        if (!rc) rc = d->sync();
        for (auto &w : ws) free_weight(d, &w);
    } else if (nm == "copy" && n_args >= 1) {
        size_t bytes = (size_t)args[0];
        DevBuf A(d), Bf(d);
        rc = A.alloc(bytes);
        if (!rc) rc = Bf.alloc(bytes);
        if (!rc) rc = rd_hip_ok(d->hip, d->hip->MemsetAsync(A.p, 1, bytes, d->stream), "memset") ? RD_OK : RD_ERR_HIP;
        for (int i = 0; i < warmup + iters && !rc; i++) {
            if (i >= warmup) (void)d->hip->EventRecord(ev[2 * (size_t)(i - warmup)], d->stream);
            rc = d->launch(d->k.copy16, 4096, 1, 1, 256, (const void *)A.p, Bf.p, (size_t)(bytes / 16));
            if (i >= warmup) (void)d->hip->EventRecord(ev[2 * (size_t)(i - warmup) + 1], d->stream);
        }
        if (!rc) rc = d->sync();
    } else if (nm == "issue" && n_args >= 3) {
        const int mode = (int)args[0], waves = (int)args[1], its = (int)args[2];
        const int cus = n_args >= 4 ? (int)args[3] : 256; // the MI355X's compute units
        if (mode < 0 || mode > 3 || waves < 1 || waves > 2 || its < 1 || its > 1000000 || cus < 1 || cus > 1024) {
            rd_set_error("issue bench: mode 0..3, waves 1..2, iterations 1..1000000, compute units 1..1024");
            rc = RD_ERR_ARG;
        }
        DevBuf In(d), Out(d);
        if (!rc) rc = In.alloc(4096);
        if (!rc) rc = Out.alloc(sizeof(float) * 256 * (size_t)cus * waves);
        if (!rc) rc = d->launch(d->k.fill_f32, 4, 1, 1, 256, In.as<float>(), (size_t)1024, 3u); // any bits do: the loop reads them as ints
        const hipFunction_t f = mode == 0 ? d->k.issue_mfma_i8 : (mode == 1 ? d->k.issue_mfma_f32 : (mode == 2 ? d->k.issue_valu : d->k.issue_all));
        for (int i = 0; i < warmup + iters && !rc; i++) {
            if (i >= warmup) (void)d->hip->EventRecord(ev[2 * (size_t)(i - warmup)], d->stream);
            rc = d->launch(f, (unsigned)(cus * waves), 1, 1, 256, its, (const int *)In.p, Out.as<float>());
            if (i >= warmup) (void)d->hip->EventRecord(ev[2 * (size_t)(i - warmup) + 1], d->stream);
        }
        if (!rc) rc = d->sync();
    } else if (nm == "topk" && n_args >= 3) {
        // args {rows, V, k[, bell]}: the top-K reduction (with Z) of `rows` logits rows of uniform values, or (bell) of sums of
        // twelve uniforms, the shape of real logits: a thin upper tail
        int rows = (int)args[0], V = (int)args[1], k = (int)args[2];
        if (rows < 1 || rows > 4096 || V < 1 || k < 1 || k > TOPK_MAX || k > V) {
            rd_set_error("topk bench: bad shape");
            rc = RD_ERR_ARG;
        }
        DevBuf L(d), I(d), Vv(d), Z(d);
        if (!rc) rc = L.alloc(sizeof(float) * (size_t)rows * V);
        if (!rc) rc = I.alloc(sizeof(int) * (size_t)rows * k);
        if (!rc) rc = Vv.alloc(sizeof(float) * (size_t)rows * k);
        if (!rc) rc = Z.alloc(sizeof(double) * (size_t)rows);
        if (!rc && n_args >= 4 && args[3]) {
            std::vector<float> h((size_t)rows * V);
            uint64_t s = 0x9E3779B97F4A7C15ULL;
            for (auto &x : h) {
                float a = -6.f;
                for (int j = 0; j < 12; j++) {
                    s ^= s << 13, s ^= s >> 7, s ^= s << 17;
                    a += (float)(s >> 40) * (1.0f / 16777216.0f);
                }
                x = 3.f * a;
            }
            rc = d->h2d(L.p, h.data(), sizeof(float) * h.size());
            if (!rc) rc = d->sync();
        } else if (!rc) {
            rc = d->launch(d->k.fill_f32, 1024, 1, 1, 256, L.as<float>(), (size_t)rows * V, 31u);
        }
        TopkScratch sc;
        if (!rc) rc = topk_scratch_alloc(d, rows, V, &sc);
        for (int i = 0; i < warmup + iters && !rc; i++) {
            if (i >= warmup) (void)d->hip->EventRecord(ev[2 * (size_t)(i - warmup)], d->stream);
            rc = launch_topk(d, (const float *)L.p, rows, V, k, 1.f, false, sc, I.as<int>(), Vv.as<float>(), Z.as<double>());
            if (i >= warmup) (void)d->hip->EventRecord(ev[2 * (size_t)(i - warmup) + 1], d->stream);
        }
        if (!rc) rc = d->sync();
        for (void *p : {(void *)sc.ghist, (void *)sc.ccount, (void *)sc.gmax, (void *)sc.cand_i, (void *)sc.cand_v, (void *)sc.invT, (void *)sc.zpart})
            if (p) d->release(p);
    } else if (nm == "moe_gemm" && n_args >= 7) {
        // args {N, K, nE, active, T, per_expert_panels, copies[, first[, bitmap[, rows]]]}: the grouped expert GEMM over nE experts of which `active`
        // have a token (spread evenly, or the first `active` ones when `first` is set: then every block with work precedes every
        // block without in dispatch order; `bitmap`: the kernel gets the active-expert bitmap and orders the grid itself; `rows`: tokens per active expert, default 1); int4 group-32 weights of arbitrary bits, `copies` weight sets used round-robin.
        int N = (int)args[0], K = (int)args[1], nE = (int)args[2], active = (int)args[3], T = (int)args[4], perE = (int)args[5];
        int copies = (int)std::max<int64_t>(1, args[6]);
        if (N <= 0 || N % 32 || K <= 0 || K % 32 || nE < 1 || nE > 256 || active < 0 || active > nE || T < 1 || T > 32) {
            rd_set_error("moe_gemm bench: bad shape");
            rc = RD_ERR_ARG;
        }
        const int nKB = (K + 255) / 256;
        const size_t wStride = (size_t)(N / 32) * nKB * 4608, wBytes = wStride * nE;
        const size_t xpStride = a8_bytes(K);
        DevBuf W(d), Xp(d), R(d), O(d), Bits(d);
        if (!rc) rc = W.alloc(wBytes * copies);
        if (!rc) rc = Xp.alloc(xpStride * (perE ? nE : 1));
        if (!rc) rc = R.alloc((size_t)32 * nE);
        if (!rc) rc = O.alloc(sizeof(float) * (size_t)T * N * 8);
        if (!rc) rc = d->launch(d->k.fill_f16, 2048, 1, 1, 256, W.as<uint16_t>(), wBytes * copies / 2, 21u);
        if (!rc) rc = d->launch(d->k.fill_f16, 256, 1, 1, 256, Xp.as<uint16_t>(), xpStride * (perE ? nE : 1) / 2, 22u);
        if (!rc) {
            std::vector<signed char> rk((size_t)32 * nE, -1);
            const int rowsPer = n_args >= 10 ? (int)std::min<int64_t>(T, std::max<int64_t>(1, args[9])) : 1;
            for (int e = 0; e < nE; e++)
                if (n_args >= 8 && args[7] ? e < active : (long)(e + 1) * active / nE > (long)e * active / nE)
                    for (int j = 0; j < rowsPer; j++) rk[(size_t)((e + j) % T) * nE + e] = 0;
            rc = d->h2d(R.p, rk.data(), rk.size());
            unsigned bits[8] = {0, 0, 0, 0, 0, 0, 0, 0};
            for (int e = 0; e < nE; e++)
                if (rk[(size_t)(e % T) * nE + e] == 0) bits[e >> 5] |= 1u << (e & 31);
            if (!rc) rc = Bits.alloc(sizeof(bits));
            if (!rc) rc = d->h2d(Bits.p, bits, sizeof(bits));
        }
        if (!rc) rc = d->sync();
        for (int i = 0; i < warmup + iters && !rc; i++) {
            const uint8_t *w = (const uint8_t *)W.p + (size_t)(i % copies) * wBytes;
            if (i >= warmup) (void)d->hip->EventRecord(ev[2 * (size_t)(i - warmup)], d->stream);
            rc = d->launch_lds(d->k.moe_gemv_w4a8, moe_gemv_grid(N, K), (unsigned)nE, 1, MOE_THREADS, moe_gemv_lds(K), (const void *)w, wStride, (const void *)Xp.p,
                           perE ? xpStride : (size_t)0, O.as<float>(), N, K, T, 1, (const signed char *)R.p, nE,
                           (n_args >= 9 && args[8]) ? (const unsigned *)Bits.p : (const unsigned *)nullptr);
            if (i >= warmup) (void)d->hip->EventRecord(ev[2 * (size_t)(i - warmup) + 1], d->stream);
        }
        if (!rc) rc = d->sync();
    } else {
        rd_set_error("rd_bench_kernel: unknown kernel '%s'", name);
        rc = RD_ERR_ARG;
    }
    for (int i = 0; i < iters; i++) {
        float ms = 0.f;
        if (!rc) (void)d->hip->EventElapsedTime(&ms, ev[2 * (size_t)i], ev[2 * (size_t)i + 1]);
        ms_out[i] = ms;
    }
    for (auto &e : ev) (void)d->hip->EventDestroy(e);
    return rc;
}

// The ragged flash-decode attention of one layer over a synthetic paged f16 KV pool (uniform [-2,2) values, scattered
// block table), rows in groups of 32 as the step batches them. ms_total[iters]: the whole call (partial + combine kernels
// of every group); ms_partial[iters] (may be NULL): the partial kernels alone. HIP events on the launch stream.
static int bench_attn_typed(rd_device *d, int kv_type, int n_seq, const int *len, int n_h, int n_kv, int hd, float scale, float softcap, int warmup,
                            int iters, float *ms_total, float *ms_partial) {
    if (!d || !len || n_seq <= 0 || iters <= 0 || !ms_total) return RD_ERR_ARG;
    if (n_kv <= 0 || n_h % n_kv || n_h / n_kv > 16 || (hd != 64 && hd != 128)) {
        rd_set_error("rd_bench_attn declines: head_dim must be 64 or 128 and the GQA group <= 16");
        return RD_DECLINED;
    }
    const int qd = n_h * hd, G = n_h / n_kv;
    int maxBlocks = 0;
    long totalBlocks = 0;
    for (int i = 0; i < n_seq; i++) {
        if (len[i] <= 0) return RD_ERR_ARG;
        int nb = (len[i] + 63) / 64;
        maxBlocks = std::max(maxBlocks, nb), totalBlocks += nb;
    }
    std::vector<int> tab((size_t)n_seq * maxBlocks, 0);
    {
        long nb = totalBlocks, stride = std::max(1L, (long)(nb * 0.618));
        while (stride < nb && std::gcd(stride, nb) != 1) stride++;
        if (stride >= nb) stride = 1;
        long idx = 0;
        for (int i = 0; i < n_seq; i++)
            for (int b = 0; b < (len[i] + 63) / 64; b++, idx++) tab[(size_t)i * maxBlocks + b] = 1 + (int)((idx * stride) % nb);
    }
    const bool i8 = kv_type == RD_KV_I8;
    // the int8 pool is filled as binary16 values over half as many elements: every byte pattern is a valid code
    const size_t poolHalves = (size_t)(totalBlocks + 1) * n_kv * 64 * hd / (i8 ? 2 : 1), scFloats = (size_t)(totalBlocks + 1) * n_kv * 64;
    DevBuf Kp(d), Vp(d), Ksc(d), Vsc(d), T(d), Q(d), O(d);
    RC(Kp.alloc(poolHalves * 2));
    RC(Vp.alloc(poolHalves * 2));
    if (i8) {
        RC(Ksc.alloc(scFloats * sizeof(float)));
        RC(Vsc.alloc(scFloats * sizeof(float)));
        RC(d->launch(d->k.fill_f32, 256, 1, 1, 256, Ksc.as<float>(), scFloats, 14u));
        RC(d->launch(d->k.fill_f32, 256, 1, 1, 256, Vsc.as<float>(), scFloats, 15u));
    }
    RC(T.alloc(sizeof(int) * tab.size()));
    RC(Q.alloc(sizeof(float) * (size_t)n_seq * qd));
    RC(O.alloc(sizeof(float) * (size_t)n_seq * qd));
    RC(d->h2d(T.p, tab.data(), sizeof(int) * tab.size()));
    RC(d->launch(d->k.fill_f16, 2048, 1, 1, 256, Kp.as<uint16_t>(), poolHalves, 11u));
    RC(d->launch(d->k.fill_f16, 2048, 1, 1, 256, Vp.as<uint16_t>(), poolHalves, 12u));
    RC(d->launch(d->k.fill_f32, 256, 1, 1, 256, Q.as<float>(), (size_t)n_seq * qd, 13u));
    struct Group {
        int r0, rows, nItems;
        DevBuf L, S, I, St, P;
        Group(rd_device *dv) : r0(0), rows(0), nItems(0), L(dv), S(dv), I(dv), St(dv), P(dv) {}
    };
    std::vector<std::unique_ptr<Group>> groups;
    for (int r0 = 0; r0 < n_seq; r0 += 32) {
        auto g = std::make_unique<Group>(d);
        g->r0 = r0, g->rows = std::min(32, n_seq - r0);
        std::vector<AttnItemH> items;
        std::vector<int> start, slots((size_t)g->rows), lens((size_t)g->rows);
        for (int i = 0; i < g->rows; i++) slots[(size_t)i] = r0 + i, lens[(size_t)i] = len[r0 + i];
        build_attn_worklist(lens.data(), nullptr, G, g->rows, n_kv, items, start);
        attn_pad_items(items); // launched as the step launches it
        g->nItems = (int)items.size();
        RC(g->L.alloc(sizeof(int) * lens.size()));
        RC(g->S.alloc(sizeof(int) * slots.size()));
        RC(g->I.alloc(sizeof(AttnItemH) * items.size()));
        RC(g->St.alloc(sizeof(int) * start.size()));
        RC(g->P.alloc(sizeof(float) * items.size() * G * (hd + 2)));
        RC(d->h2d(g->L.p, lens.data(), sizeof(int) * lens.size()));
        RC(d->h2d(g->S.p, slots.data(), sizeof(int) * slots.size()));
        RC(d->h2d(g->I.p, items.data(), sizeof(AttnItemH) * items.size()));
        RC(d->h2d(g->St.p, start.data(), sizeof(int) * start.size()));
        groups.push_back(std::move(g));
    }
    RC(d->sync());
    const size_t nG = groups.size();
    std::vector<hipEvent_t> ev((size_t)iters * 2), evp((size_t)iters * nG * 2);
    for (auto &e : ev) HIPCHK(EventCreate(&e));
    for (auto &e : evp) HIPCHK(EventCreate(&e));
    int rc = RD_OK;
    for (int i = 0; i < warmup + iters && !rc; i++) {
        const bool timed = i >= warmup;
        const size_t t = (size_t)(i - warmup);
        if (timed) (void)d->hip->EventRecord(ev[2 * t], d->stream);
        for (size_t gi = 0; gi < nG && !rc; gi++) {
            Group &g = *groups[gi];
            if (timed) (void)d->hip->EventRecord(evp[(t * nG + gi) * 2], d->stream);
            if (i8)
                rc = d->launch(d->k.attn_partial_i8, (unsigned)g.nItems, 1, 1, 64, (const void *)g.I.p, (const int *)g.L.p, (const int *)g.S.p, (const int *)T.p,
                               maxBlocks, (const signed char *)Kp.p, (const signed char *)Vp.p, (const float *)Ksc.p, (const float *)Vsc.p,
                               (const float *)((const float *)Q.p + (size_t)g.r0 * qd), g.P.as<float>(), n_h, n_kv, hd, scale, softcap, 0);
            else {
                const AttnLaunch al = attn_partial_kernel(d, false, false, (size_t)g.nItems);
                rc = d->launch(al.f, (unsigned)g.nItems / al.waves, 1, 1, 64 * al.waves, (const void *)g.I.p, (const int *)g.L.p, (const int *)g.S.p, (const int *)T.p, maxBlocks,
                               (const uint16_t *)Kp.p, (const uint16_t *)Vp.p, (const float *)((const float *)Q.p + (size_t)g.r0 * qd), g.P.as<float>(), n_h, n_kv, hd,
                               scale, softcap, 0);
            }
            if (timed) (void)d->hip->EventRecord(evp[(t * nG + gi) * 2 + 1], d->stream);
            if (!rc)
                rc = d->launch(d->k.attn_combine, (unsigned)n_h, (unsigned)g.rows, 1, (unsigned)(ATTN_PIECES * hd / 4), (const float *)g.P.p, (const int *)g.St.p, G,
                               (float *)((float *)O.p + (size_t)g.r0 * qd), n_h, n_kv, hd, (const float *)nullptr);
        }
        if (timed) (void)d->hip->EventRecord(ev[2 * t + 1], d->stream);
    }
    if (!rc) rc = d->sync();
    for (int i = 0; i < iters; i++) {
        float ms = 0.f, mp = 0.f;
        if (!rc) {
            (void)d->hip->EventElapsedTime(&ms, ev[2 * (size_t)i], ev[2 * (size_t)i + 1]);
            for (size_t gi = 0; gi < nG; gi++) {
                float x = 0.f;
                (void)d->hip->EventElapsedTime(&x, evp[((size_t)i * nG + gi) * 2], evp[((size_t)i * nG + gi) * 2 + 1]);
                mp += x;
            }
        }
        ms_total[i] = ms;
        if (ms_partial) ms_partial[i] = mp;
    }
    for (auto &e : ev) (void)d->hip->EventDestroy(e);
    for (auto &e : evp) (void)d->hip->EventDestroy(e);
    return rc;
}
extern "C" int rd_bench_attn(rd_device *d, int n_seq, const int *len, int n_h, int n_kv, int hd, float scale, float softcap, int warmup, int iters,
                             float *ms_total, float *ms_partial) {
    return bench_attn_typed(d, RD_KV_F16, n_seq, len, n_h, n_kv, hd, scale, softcap, warmup, iters, ms_total, ms_partial);
}
extern "C" int rd_bench_attn_i8(rd_device *d, int n_seq, const int *len, int n_h, int n_kv, int hd, float scale, float softcap, int warmup, int iters,
                                float *ms_total, float *ms_partial) {
    return bench_attn_typed(d, RD_KV_I8, n_seq, len, n_h, n_kv, hd, scale, softcap, warmup, iters, ms_total, ms_partial);
}
