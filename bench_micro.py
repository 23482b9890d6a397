"""The other measurement configurations of the decode path (bench.py --workload c2|c3|c5|kquant): one JSON line each, same form as
the default workload's. Inputs are synthetic and resident in HBM before the timed region; times are HIP events on the launch
stream; bytes are the algorithmic bytes of the call (every weight byte once, every KV byte once per sequence)."""
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
T0 = time.time()


def log(msg):
    print("[bench %6.1fs] %s" % (time.time() - T0, msg), file=sys.stderr, flush=True)


def threads():
    return min(16, len(os.sched_getaffinity(0)))


def emit(out):
    print(json.dumps(out, default=float))


def base_line(metric, value, unit, steps, warmup, ms, workload, data, extra_cfg=None, dtype="i8"):
    cfg = {"workload": workload}
    cfg.update(extra_cfg or {})
    return {"metric": metric, "value": round(value, 1), "unit": unit, "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype, "data": data,
            "config": cfg}


# ------------------------------------------------------------------------------------------------------------ C2
def host_cpu():
    """(model name, physical cores) of this host from /proc/cpuinfo: distinct (physical id, core id) pairs, so SMT siblings
    count once; (None, None) where the file does not say."""
    model, cores, phys, core = None, set(), None, None
    try:
        for line in open("/proc/cpuinfo"):
            k, _, v = line.partition(":")
            k, v = k.strip(), v.strip()
            if k == "model name" and model is None:
                model = v
            elif k == "physical id":
                phys = v
            elif k == "core id":
                core = v
            elif not k and phys is not None and core is not None:
                cores.add((phys, core))
                phys = core = None
        if phys is not None and core is not None:
            cores.add((phys, core))
    except OSError:
        pass
    return model, (len(cores) or None)


def counter_traffic(key, algorithmic_bytes):
    """HBM bytes per launch of a kernel for THIS run: the run's algorithmic bytes times the ratio (counter traffic / algorithmic
    bytes) that the rocprofv3 counter runs recorded for the kernel on this workload (profiles/traffic.json names the run each
    ratio comes from). Returns (traffic, ratio, source) or (None, None, None)."""
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if not os.path.exists(tpath):
        return None, None, None
    e = json.load(open(tpath)).get(key)
    if not e:
        return None, None, None
    return int(round(e["ratio"] * algorithmic_bytes)), e["ratio"], e["source"]


def cpu_fields(n_threads):
    """The fields of a cpu_baseline block that say what it ran on: threads used (`cores`, as the bench contract names them), the
    host's CPU model and its physical core count."""
    model, phys = host_cpu()
    return {"cores": n_threads, "threads": n_threads, "physical_cores_on_host": phys, "cpu_model": model}


def run_c2(args):
    """Q4_K dequant-GEMM: up 14336x4096, down 4096x14336, fused gate|up + SwiGLU + quantization; M in {1,4,16,32,64}.
    A step is one GEMM call (M = 64 is two passes of 32 rows, as the step batches rows)."""
    from goinfer_amd import capi
    steps, warmup = (args.steps if args.steps != 128 else 100), (args.warmup if args.warmup != 8 else 20)
    dev = capi.Device(0)
    W = 14336 * (4096 // 256) * 144
    cases = []
    for name, kern, N, K, wbytes in (("up 14336x4096", "gemm_q4k", 14336, 4096, W), ("down 4096x14336", "gemm_q4k", 4096, 14336, W),
                                     ("fused gate|up 2x14336x4096 + SwiGLU", "gateup", 14336, 4096, 2 * W)):
        for M in ((args.m,) if getattr(args, "m", 0) else (1, 4, 16, 32, 64)):
            ms = dev.bench_kernel(kern, [N, K, M, 8], warmup, steps)  # 8 weight copies round-robin: nothing stays in the 256 MB cache
            t = float(np.median(ms))
            nbytes = wbytes + 4 * M * K + (4 * M * N if kern == "gemm_q4k" else 2 * M * N)  # weights + activations in + result out
            flops = 2.0 * M * N * K * (2 if kern == "gateup" else 1)
            cases.append({"case": name, "M": M, "us": round(t * 1e3, 2), "GBs": round(nbytes / t / 1e6, 1), "TFLOPs": round(flops / t / 1e9, 1),
                          "bytes": int(nbytes)})
            log("%s M=%d: %.1f us, %.0f GB/s" % (name, M, t * 1e3, nbytes / t / 1e6))
    head = next(c for c in cases if c["case"].startswith("fused") and c["M"] == (getattr(args, "m", 0) or 32))
    out = base_line("Q4_K dequant-GEMM achieved HBM GB/s (fused gate|up SwiGLU at M=32; all cases listed)", head["GBs"], "GB/s", steps, warmup,
                    head["us"] / 1e3, "configs[1]: Q4_K GEMM 14336x4096 / 4096x14336 / fused gate|up, M in {1,4,16,32,64}",
                    "synthetic: random Q4_K super-blocks with sane f16 scales, 8 weight copies used round-robin", {"cases": cases})
    out["roofline"] = {"bound": "hbm", "achieved": head["GBs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(head["GBs"] / HBM_PEAK_GBS, 4),
                       "kernel": "rd_k_gemm8_q4k_gateup", "avg_launch_ms": round(head["us"] / 1e3, 5), "algorithmic_bytes_per_launch": head["bytes"]}
    out["roofline"]["traffic"], out["roofline"]["traffic_ratio"], out["roofline"]["traffic_source"] = counter_traffic(
        "gemm8_q4k_gateup/ffn-14336x4096-m32", head["bytes"])
    cpu = None
    if not args.no_cpu:
        from goinfer_amd import synth
        from oracle import binding as ob
        ob.set_threads(threads())
        g, u = synth.q4k_normal(1, 14336, 4096), synth.q4k_normal(2, 14336, 4096)
        wg, wu = ob.WMat(ob.OR_Q4K, 14336, 4096, g, act_group=32), ob.WMat(ob.OR_Q4K, 14336, 4096, u, act_group=32)
        a = synth.normal(3, 32 * 4096, 1.0).reshape(32, 4096)
        ob.swiglu(ob.matmul(wg, a), ob.matmul(wu, a))
        n, t = 0, 0.0
        while t < 10.0 and n < 400:
            t0 = time.time()
            ob.swiglu(ob.matmul(wg, a), ob.matmul(wu, a))
            t += time.time() - t0
            n += 1
        cpu = {"value": round(head["bytes"] / (t / n) / 1e9, 2), "unit": "GB/s", **cpu_fields(threads()), "kind": "port",
               "sample": "oracle gate and up matmuls + SwiGLU at M=32, %d calls (%.1f s)" % (n, t)}
    out["cpu_baseline"] = cpu
    dev.close()
    emit(out)


def run_kquant(args):
    """The Q5_K and Q6_K lanes beside Q4_K: dequant-GEMMs at the FFN shapes and at the 128256 x 4096 head (the tensor GGUF
    Q4_K_M files most often store as Q6_K), M = 1 and 32. Bytes are the file's own super-blocks + activations in + result out."""
    from goinfer_amd import capi
    steps, warmup = (args.steps if args.steps != 128 else 60), (args.warmup if args.warmup != 8 else 10)
    dev = capi.Device(0)
    cases = []
    for kern, bb in (("gemm_q4k", 144), ("gemm_q5k", 176), ("gemm_q6k", 210)):
        for N, K in ((14336, 4096), (4096, 14336), (128256, 4096)):
            for M in (1, 32):
                ms = dev.bench_kernel(kern, [N, K, M, 4 if N > 100000 else 8], warmup, steps)
                t = float(np.median(ms))
                nbytes = N * (K // 256) * bb + 4 * M * K + 4 * M * N
                cases.append({"kernel": "rd_k_gemm8_" + kern[5:], "N": N, "K": K, "M": M, "us": round(t * 1e3, 2), "GBs": round(nbytes / t / 1e6, 1), "bytes": int(nbytes)})
                log("%s %dx%d M=%d: %.1f us, %.0f GB/s" % (kern, N, K, M, t * 1e3, nbytes / t / 1e6))
    head = next(c for c in cases if c["kernel"] == "rd_k_gemm8_q6k" and c["N"] == 128256 and c["M"] == 32)
    out = base_line("Q6_K dequant-GEMM achieved HBM GB/s (head 128256x4096 at M=32; all cases listed)", head["GBs"], "GB/s", steps, warmup,
                    head["us"] / 1e3, "Q4_K / Q5_K / Q6_K GEMM at 14336x4096, 4096x14336, 128256x4096, M in {1,32}",
                    "synthetic: random super-blocks with sane f16 scales, 4-8 weight copies used round-robin", {"cases": cases}, dtype="i8")
    out["roofline"] = {"bound": "hbm", "achieved": head["GBs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(head["GBs"] / HBM_PEAK_GBS, 4),
                       "traffic": None, "kernel": "rd_k_gemm8_q6k_kw2", "avg_launch_ms": round(head["us"] / 1e3, 5),
                       "algorithmic_bytes_per_launch": head["bytes"]}
    cpu = None
    if not args.no_cpu:
        from goinfer_amd import synth
        from oracle import binding as ob
        ob.set_threads(threads())
        N, K = 16384, 4096  # a bounded slice of the head's rows
        w = ob.WMat(ob.OR_Q6K, N, K, synth.kquant_normal("q6k", 1, N, K), act_group=32)
        a = synth.normal(3, 32 * K, 1.0).reshape(32, K)
        ob.matmul(w, a)
        n, t = 0, 0.0
        while t < 10.0 and n < 400:
            t0 = time.time()
            ob.matmul(w, a)
            t += time.time() - t0
            n += 1
        cpu = {"value": round((N * (K // 256) * 210 + 4 * 32 * (K + N)) / (t / n) / 1e9, 2), "unit": "GB/s", **cpu_fields(threads()), "kind": "port",
               "sample": "oracle Q6_K matmul, %d x %d rows of the head at M=32, %d calls (%.1f s)" % (N, K, n, t)}
    out["cpu_baseline"] = cpu
    dev.close()
    emit(out)


def run_topk(args):
    """The device-side top-K of logits rows (goinfer's TopKRow): rows of bell-shaped values, as logits are, and of uniform ones,
    whose crowded threshold bin sends them down the exact one-block route. A step is one reduction of all the rows, Z included."""
    from goinfer_amd import capi
    steps, warmup = (args.steps if args.steps != 128 else 50), (args.warmup if args.warmup != 8 else 10)
    dev = capi.Device(0)
    cases = []
    for rows, V, k in ((1, 128256, 256), (32, 128256, 256), (32, 128256, 1024), (128, 128256, 256), (32, 151936, 256), (32, 262144, 1024)):
        for bell in (1, 0):
            ms = dev.bench_kernel("topk", [rows, V, k, bell], warmup, steps)
            t = float(np.median(ms))
            cases.append({"rows": rows, "V": V, "k": k, "values": "bell" if bell else "uniform", "us": round(t * 1e3, 1),
                          "GBs": round(rows * V * 4 / t / 1e6, 1), "bytes": rows * V * 4})
            log("%d rows x %d, k=%d, %s: %.1f us" % (rows, V, k, "bell" if bell else "uniform", t * 1e3))
    head = next(c for c in cases if c["rows"] == 32 and c["V"] == 128256 and c["k"] == 256 and c["values"] == "bell")
    out = base_line("device-side top-K of logits rows, achieved GB/s over one read of the rows (32 rows of 128256, K=256; all cases listed)",
                    head["GBs"], "GB/s", steps, warmup, head["us"] / 1e3, "top-K of logits rows (TopKRow): ids, logits and Z",
                    "synthetic: sums of twelve uniforms (bell) or uniform values", {"cases": cases}, dtype="f32")
    out["roofline"] = {"bound": "hbm", "achieved": head["GBs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(head["GBs"] / HBM_PEAK_GBS, 4),
                       "traffic": None, "kernel": "rd_k_topk_hist + rd_k_topk_pick + rd_k_topk_finish", "avg_launch_ms": round(head["us"] / 1e3, 5),
                       "algorithmic_bytes_per_launch": head["bytes"]}
    cpu = None
    if not args.no_cpu:
        from oracle import binding as ob
        rng = np.random.default_rng(1)
        x = (rng.standard_normal((32, 128256)) * 3).astype(np.float32)
        n, t = 0, 0.0
        while t < 5.0 and n < 200:
            t0 = time.time()
            for r in range(32):
                ob.topk_by_logit(x[r], 256)
                ob.softmax_z(x[r], 0.7)
            t += time.time() - t0
            n += 1
        cpu = {"value": round(32 * 128256 * 4 / (t / n) / 1e9, 2), "unit": "GB/s", **cpu_fields(1), "kind": "port",
               "sample": "oracle topKByLogit + Z over 32 rows of 128256, K=256, %d passes (%.1f s)" % (n, t)}
    out["cpu_baseline"] = cpu
    dev.close()
    emit(out)


def run_issue(args):
    """What one SIMD sustains of the int8 GEMMs' inner-loop instruction mix with no memory in the loop (rd_k_issue_*): the eight int8
    MFMAs, the eight f32 MFMAs and the fold's 256 vector instructions of one (32 x 32 x 256) tile-block, each alone and all together,
    at one and two waves a SIMD. `overlap` is the part of the shorter of (matrix core, vector ALU) that the mix hides:
    0 = the times add, 1 = the shorter one is free. A step is one launch of `its` iterations on every SIMD."""
    from goinfer_amd import capi
    steps, warmup = (args.steps if args.steps != 128 else 7), (args.warmup if args.warmup != 8 else 2)
    its = 20000
    dev = capi.Device(0)
    cases = []
    for waves in (1, 2):
        ns = {}
        for mode, name in enumerate(("mfma_i8", "mfma_f32", "valu", "all")):
            ms = dev.bench_kernel("issue", [mode, waves, its], warmup, steps)
            ns[name] = float(np.median(ms)) * 1e6 / its / waves  # the SIMD's time per tile-block
            log("%d wave(s) a SIMD, %s: %.1f ns per tile-block" % (waves, name, ns[name]))
        mf = ns["mfma_i8"] + ns["mfma_f32"]
        hidden = (mf + ns["valu"] - ns["all"]) / min(mf, ns["valu"])
        cases.append({"waves_per_simd": waves, **{k + "_ns": round(v, 1) for k, v in ns.items()}, "sum_ns": round(mf + ns["valu"], 1), "overlap": round(hidden, 3)})
    two = cases[-1]
    tops = 2 * 8 * 32 * 32 * 32 / two["all_ns"] * 1024 / 1e3  # int8 multiply-adds x 2 of a tile-block, on 1024 SIMDs, TOP/s
    out = base_line("int8 TOP/s of the Q4_K tile-block's instruction mix at two waves a SIMD, no memory in the loop", round(tops, 1), "TOP/s", steps, warmup,
                    two["all_ns"] * its * 2 / 1e6, "issue-rate probe: 8 int8 MFMAs + 8 f32 MFMAs + 256 fold instructions a tile-block",
                    "synthetic: registers only", {"cases": cases, "iterations": its}, dtype="i8")
    out["roofline"] = {"bound": "mfma", "achieved": round(tops, 1), "peak": 5000.0, "unit": "TOP/s", "frac": round(tops / 5000.0, 4), "traffic": None,
                       "kernel": "rd_k_issue_all", "avg_launch_ms": round(two["all_ns"] * its * 2 / 1e6, 4)}
    out["cpu_baseline"] = None
    dev.close()
    emit(out)


# ------------------------------------------------------------------------------------------------------------ C3
def run_c3(args):
    """Ragged flash-decode attention: 64 sequences, KV lengths U[128,8192], 32 Q / 8 KV heads, head_dim 128, f16 KV; once without
    softcap and once with softcap 50. A step is one ragged call (one layer)."""
    from goinfer_amd import capi
    steps, warmup = (args.steps if args.steps != 128 else 100), (args.warmup if args.warmup != 8 else 20)
    nH, nKV, hd, nseq = 32, 8, 128, 64
    lens = np.random.default_rng(args.seed).integers(128, 8193, nseq).astype(np.int32)
    scale = float(1.0 / np.sqrt(hd))
    kv = getattr(args, "kv", "f16")
    kv_bytes = float(lens.sum()) * 2 * nKV * (hd * 2 if kv == "f16" else hd + 4)  # int8: the codes and one f32 scale per (position, kv head)
    io_bytes = 2 * nseq * nH * hd * 4
    dev = capi.Device(0)
    res = {}
    for cap in (0.0, 50.0):
        tot, part = dev.bench_attn(lens, nH, nKV, hd, scale, cap, warmup, steps, kv=kv)
        res[cap] = (float(np.median(tot)), float(np.median(part)))
        log("softcap %g: call %.1f us (%.0f GB/s), partial kernels %.1f us (%.0f GB/s)" % (
            cap, res[cap][0] * 1e3, (kv_bytes + io_bytes) / res[cap][0] / 1e6, res[cap][1] * 1e3, kv_bytes / res[cap][1] / 1e6))
    t, tp = res[0.0]
    gbs = (kv_bytes + io_bytes) / t / 1e6
    out = base_line("ragged flash-decode attention achieved HBM GB/s (64 sequences, KV U[128,8192], 32/8 heads, head_dim 128)", gbs, "GB/s", steps,
                    warmup, t, "configs[2]: ragged attention microbench" + ("" if kv == "f16" else " (variant: int8 KV cache)"),
                    "synthetic: uniform [-2,2) f16 KV (or random int8 codes and scales) in a paged pool with a scattered block table, f32 q",
                    {"kv": kv, "n_seq": nseq, "kv_positions": int(lens.sum()), "kv_len_min": int(lens.min()), "kv_len_max": int(lens.max()), "seed": args.seed,
                     "cases": [{"softcap": c, "call_us": round(v[0] * 1e3, 2), "call_GBs": round((kv_bytes + io_bytes) / v[0] / 1e6, 1),
                                "partial_kernels_us": round(v[1] * 1e3, 2), "partial_kernels_GBs": round(kv_bytes / v[1] / 1e6, 1)} for c, v in res.items()]}, dtype="f16")
    # the partial kernel is launched once per group of 32 rows: two launches per call here
    per_launch = (kv_bytes + nseq * nH * hd * 4) / 2
    out["roofline"] = {"bound": "hbm", "achieved": round(per_launch / (tp / 2) / 1e6, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                       "frac": round(per_launch / (tp / 2) / 1e6 / HBM_PEAK_GBS, 4),
                       "kernel": "rd_k_attn_partial_wide" if kv == "f16" else "rd_k_attn_partial_i8",
                       "avg_launch_ms": round(tp / 2, 5), "algorithmic_bytes_per_launch": int(per_launch)}
    out["roofline"]["traffic"], out["roofline"]["traffic_ratio"], out["roofline"]["traffic_source"] = counter_traffic(
        "attn_partial/64seq-u128-8192/%s" % kv, per_launch)
    cpu = None
    if not args.no_cpu:
        from goinfer_amd import synth
        from oracle import binding as ob
        ob.set_threads(threads())
        pick = list(range(0, nseq, 8))
        kvd = nKV * hd
        ops = []
        for i in pick:
            n = int(lens[i])
            ops.append((synth.normal(990 + i, nH * hd, 1.0), ob.f16_round_trip(synth.normal(900 + i, n * kvd, 1.0).reshape(n, kvd)),
                        ob.f16_round_trip(synth.normal(950 + i, n * kvd, 1.0).reshape(n, kvd)), n))
        t_cpu, pos, reps = 0.0, 0, 0
        while t_cpu < 10.0 and reps < 2000:
            for q, k, v, n in ops:
                t0 = time.time()
                ob.attend(q, k, v, n, nH, nKV, hd, scale, 0.0)
                t_cpu += time.time() - t0
                pos += n
            reps += 1
        cpu = {"value": round(pos * 2 * kvd * 2 / t_cpu / 1e9, 3), "unit": "GB/s", **cpu_fields(threads()), "kind": "port",
               "sample": "oracle attention (f64 accumulate, heads in parallel) on %d of the %d sequences, %d passes, %d positions (%.1f s)" % (
                   len(pick), nseq, reps, pos, t_cpu)}
    out["cpu_baseline"] = cpu
    dev.close()
    emit(out)


# ------------------------------------------------------------------------------------------------------------ C5
def run_c5(args):
    """Qwen3-MoE-30B-A3B shape: 48 layers, 128 experts top-8 (int4-g32 experts, f32 router), Q4_K attention projections, int8 head;
    16 ragged slots, ctx U[256,2048], greedy decode. A step is one decode step of the batch."""
    from goinfer_amd import capi, workloads
    layers = args.layers if args.layers != 32 else 48
    B = args.batch if args.batch != 32 else 16
    steps, warmup = (args.steps if args.steps != 128 else 64), (args.warmup if args.warmup != 8 else 4)
    cfg = workloads.qwen3_moe_cfg(layers, exp_act_group=getattr(args, "exp_act_group", 0))
    row_act = cfg["exp_act_group"] == 0
    rng = np.random.default_rng(args.seed)
    lens = rng.integers(256, 2049, B).astype(np.int64)
    ids0 = rng.integers(0, cfg["vocab"], B).astype(np.int32)
    cap = int(lens.max()) + steps + warmup + 8
    dev = capi.Device(0)
    log("building %s, %d layers" % (cfg["name"], layers))
    res = workloads.Resident(dev, cfg, seed=args.seed, slots=B, ctx_cap=cap, keep_layers=0 if args.no_cpu else 1, progress=log)
    kept_kv = res.prefill_kv(lens, progress=log)
    slots = np.arange(B, dtype=np.int32)
    dev.sync()
    ms = res.model.bench_steps(slots, lens, ids0, warmup, steps)
    dev.sync()
    tok_s = B * steps / (float(ms.sum()) / 1e3)
    log("steps: %.3f ms mean, %.3f ms median" % (ms.mean(), float(np.median(ms))))
    # distinct experts per layer from the last step's recorded routing
    idx = res.model.last_moe_indices(B)  # [B][layers][k]
    distinct = [len(set(idx[:, l, :].ravel().tolist())) for l in range(layers)]
    ebytes = workloads.expert_bytes(cfg)
    mid = lens + warmup + steps // 2
    kv_pos = workloads.kv_bytes_per_position(cfg)
    kv_read = float((mid + 1).sum()) * kv_pos
    w_bytes = workloads.weight_bytes(cfg)
    exp_bytes = float(sum(distinct)) * ebytes
    step_bytes = w_bytes + exp_bytes + kv_read + B * kv_pos
    step_gbs = step_bytes / (ms.mean() / 1e3) / 1e9
    pos_prof = (lens + warmup + steps).astype(np.int32)
    prof = {}
    for rep in range(3):
        for k, (t, n) in res.model.bench_profile(slots, pos_prof + rep, ids0).items():
            a = prof.setdefault(k, [0.0, 0])
            a[0] += t
            a[1] += n
    classes = {k: {"ms_per_step": round(v[0] / 3, 4), "launches_per_step": v[1] // 3} for k, v in prof.items()}
    # dominant kernel: the experts' gate|up GEMM (one launch per layer over every touched expert; two thirds of an expert's bytes)
    idx2 = res.model.last_moe_indices(B)
    d2 = float(sum(len(set(idx2[:, l, :].ravel().tolist())) for l in range(layers)))
    g_ms = prof["moe_gemm_gateup"][0] / prof["moe_gemm_gateup"][1]
    per_launch = d2 * ebytes * (2.0 / 3.0) / layers
    gu_kernel = "rd_k_moe_gemv_w4a8r_gateup" if row_act else "rd_k_moe_gemv_w4a8_gateup"
    traffic, t_ratio, t_src = counter_traffic("%s/%s" % (gu_kernel[5:], cfg["name"]), per_launch)
    act_txt = "int8 activations per token row" if row_act else "int8 activations per group of 32 (a variant of the configuration)"
    out = base_line("batch-16 decode tok/s, Qwen3-MoE-30B-A3B shape (int4-g32 experts); achieved HBM GB/s vs peak", tok_s, "tok/s", steps, warmup,
                    float(ms.mean()), "configs[4]: %s, %d layers, B=%d ragged, ctx U[256,2048], greedy decode, experts' %s" % (cfg["name"], layers, B, act_txt),
                    "synthetic: N(0,0.02) weights (Q4_K projections, int4-g32 experts, f32 router, int8 head), N(0,1) KV, random token ids",
                    {"batch": B, "ctx_min": int(lens.min()), "ctx_max": int(lens.max()), "ctx_mean": float(lens.mean()), "seed": args.seed,
                     "distinct_experts_per_layer_mean": round(float(np.mean(distinct)), 1)})
    out["step_hbm"] = {"algorithmic_bytes_per_step": int(step_bytes), "achieved_GBs": round(step_gbs, 1), "frac_of_peak": round(step_gbs / HBM_PEAK_GBS, 4),
                       "dense_weight_bytes": int(w_bytes), "expert_bytes": int(exp_bytes), "kv_read_bytes": int(kv_read)}
    out["roofline"] = {"bound": "hbm", "achieved": round(per_launch / (g_ms / 1e3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                       "frac": round(per_launch / (g_ms / 1e3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_ratio": t_ratio, "traffic_source": t_src,
                       "kernel": gu_kernel,
                       "avg_launch_ms": round(g_ms, 5), "algorithmic_bytes_per_launch": int(per_launch)}
    out["kernel_classes"] = classes
    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline_moe(res, cfg, lens, kept_kv)
    out["cpu_baseline"] = cpu
    res.close()
    dev.close()
    emit(out)


def cpu_baseline_moe(res, cfg, lens, kept_kv):
    """The oracle's decodeMultiStep on the first layer of the same model (all 128 experts resident), the same ragged batch and KV,
    greedy steps for about ten seconds; the per-layer cost scaled to the full depth."""
    from goinfer_amd.workloads import inv_freq
    from oracle import binding as ob
    ob.set_threads(threads())
    layers = []
    for kp in res.kept:
        lw = {p: ob.WMat(ob.OR_Q4K, kp[p][1], kp[p][2], kp[p][0], act_group=32) for p in ("q", "k", "v", "o")}
        for n in ("attn_norm", "ffn_norm", "q_norm", "k_norm"):
            lw[n] = kp[n]
        lw["router"] = ob.WMat.from_f32(kp["router"])
        for proj in ("gate", "up", "down"):
            lw["exp_" + proj] = [ob.WMat(ob.OR_W4A8, ex[proj][2], ex[proj][3], ex[proj][0], ex[proj][1], act_group=cfg.get("exp_act_group", 32))
                                 for ex in kp["experts"]]
        layers.append(lw)
    nL = len(layers)
    c = dict(cfg)
    c.update(n_layers=nL, kv_f16=1)
    hq, hs = res.head
    head = ob.WMat(ob.OR_W8A8, hq.shape[0], hq.shape[1], hq, hs, act_group=32)
    om = ob.OracleModel(c, layers, res.final_norm, head, inv_freq(cfg["head_dim"], cfg["theta"]))
    B, MAXS = len(lens), 64
    caches = []
    for i, n in enumerate(lens):
        cp = om.new_cache(int(n) + MAXS + 2)
        for l in range(nL):
            k, v = kept_kv[l]
            om.cache_upload(cp, l, 0, k[:n], v[:n])
        caches.append(cp)
    emb = res.embed_rows(np.arange(B) * 977 % cfg["vocab"])
    om.step(emb, caches)
    n_steps, t_step = 0, 0.0
    while n_steps < MAXS - 1 and t_step < 10.0:
        t0 = time.time()
        logits = om.step(emb, caches)
        t_step += time.time() - t0
        n_steps += 1
        emb = res.embed_rows(np.array([ob.argmax(r) for r in logits]))
    t0 = time.time()
    for _ in range(3):
        ob.matmul(head, emb)
    t_head = (time.time() - t0) / 3
    for cp in caches:
        om.free_cache(cp)
    per_layer = max(t_step / n_steps - t_head, 1e-9) / nL
    full = per_layer * cfg["n_layers"] + t_head
    return {"value": round(B / full, 3), "unit": "tok/s", **cpu_fields(threads()), "kind": "port",
            "sample": "oracle decodeMultiStep, %d of %d layers + int8 head, B=%d at the run's context lengths, %d greedy steps (%.1f s), "
                      "per-layer cost scaled to %d layers" % (nL, cfg["n_layers"], B, n_steps, t_step, cfg["n_layers"])}


# ------------------------------------------------------------------------------------------------------------ prefill
MFMA_I8_PEAK_TOPS = 5000.0


def run_prefill(args):
    """A prompt pass into the decode step's own paged KV (PrefillLast): Llama-3-8B shape, one sequence, 2048 prompt tokens from
    position 0, in passes of the model's widest step (512 rows); token ids through the embedding table, so nothing crosses PCIe inside the timed region.
    A step is one whole prompt."""
    from goinfer_amd import capi, workloads
    n_tok = 2048
    steps, warmup = (args.steps if args.steps != 128 else 5), (args.warmup if args.warmup != 8 else 1)
    cfg = workloads.llama3_8b_cfg(args.layers)
    dev = capi.Device(0)
    log("building %s, %d layers" % (cfg["name"], args.layers))
    res = workloads.Resident(dev, cfg, seed=args.seed, slots=1, ctx_cap=n_tok + 64, keep_layers=0 if args.no_cpu else min(4, args.layers), progress=log)
    rng = np.random.default_rng(args.seed)
    ids = rng.integers(0, cfg["vocab"], n_tok).astype(np.int32)
    ms = []
    for i in range(warmup + steps):
        t = res.model.bench_prefill(0, ids)
        if i >= warmup:
            ms.append(t)
        log("prompt %d: %.2f ms" % (i, t))
    ms = np.array(ms)
    tok_s = n_tok / (float(ms.mean()) / 1e3)
    _, prof = res.model.bench_prefill(0, ids, profile=True)
    classes = {k: {"ms_per_step": round(v[0], 4), "launches_per_step": v[1]} for k, v in prof.items()}
    # dominant kernels: the many-row Q4_K GEMMs (every weight tile decoded once for four row tiles of 32); the four projections of
    # a layer are one launch each per pass. Flops over all rows of the prompt, milliseconds over all four classes
    # (the last row's one-row step rides in the same classes: 1 row of 2048).
    H, hd = cfg["hidden"], cfg["head_dim"]
    qd, kvd, I = cfg["n_heads"] * hd, cfg["n_kv"] * hd, cfg["inter"]
    w_elems = (qd + 2 * kvd) * H + H * qd + 2 * I * H + H * I
    flops = 2.0 * n_tok * w_elems * cfg["n_layers"]
    g_ms = sum(prof[k][0] for k in ("gemm_qkv", "gemm_o", "gemm_gateup", "gemm_down"))
    g_n = sum(prof[k][1] for k in ("gemm_qkv", "gemm_o", "gemm_gateup", "gemm_down"))
    tfl = flops / (g_ms / 1e3) / 1e12
    out = base_line("prompt tok/s into the paged KV, Llama-3-8B-shape Q4_K, 2048-token prompt; achieved int8 MFMA TOP/s vs peak", tok_s, "tok/s", steps, warmup,
                    float(ms.mean()), "prefill: %s, %d layers, one sequence, %d prompt tokens from position 0 (PrefillLast), passes of %d rows"
                    % (cfg["name"], args.layers, n_tok, res.model.max_rows()),
                    "synthetic: N(0,0.02) weights quantized to Q4_K (int8 head and embedding), random token ids", {"prompt_tokens": n_tok, "seed": args.seed})
    out["roofline"] = {"bound": "mfma", "achieved": round(tfl, 1), "peak": MFMA_I8_PEAK_TOPS, "unit": "TOP/s", "frac": round(tfl / MFMA_I8_PEAK_TOPS, 4),
                       "traffic": None, "kernel": "rd_k_gemm8_q4k_rows* (qkv with RoPE and KV store, o, gate|up with SwiGLU, down)", "avg_launch_ms": round(g_ms / g_n, 5),
                       "algorithmic_flops_per_launch": int(flops / g_n)}
    out["kernel_classes"] = classes
    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline_prefill(res, cfg, ids)
    out["cpu_baseline"] = cpu
    res.close()
    dev.close()
    emit(out)


def cpu_baseline_prefill(res, cfg, ids):
    """The oracle walking the first tokens of the same prompt one at a time through the first layers of the same model (the reference's CPU
    prompt pass computes the same rows), about ten seconds; the per-layer cost scaled to the full depth, the head left out as in a prompt pass."""
    from goinfer_amd.workloads import inv_freq
    from oracle import binding as ob
    ob.set_threads(threads())
    layers = []
    for kp in res.kept:
        lw = {p: ob.WMat(ob.OR_Q4K, kp[p][1], kp[p][2], kp[p][0], act_group=32) for p in ("q", "k", "v", "o", "gate", "up", "down")}
        lw["attn_norm"], lw["ffn_norm"] = kp["attn_norm"], kp["ffn_norm"]
        layers.append(lw)
    nL = len(layers)
    c = dict(cfg)
    c.update(n_layers=nL, kv_f16=1)
    hq, hs = res.head
    head = ob.WMat(ob.OR_W8A8, hq.shape[0], hq.shape[1], hq, hs, act_group=32)
    om = ob.OracleModel(c, layers, res.final_norm, head, inv_freq(cfg["head_dim"], cfg["theta"]))
    MAXT = 1024
    cp = om.new_cache(MAXT + 2)
    emb = res.embed_rows(ids[:MAXT])
    om.step(emb[0:1], [cp])
    t0 = time.time()
    for _ in range(3):
        ob.matmul(head, emb[0:1])
    t_head = (time.time() - t0) / 3
    n, t = 0, 0.0
    while n < MAXT - 1 and t < 10.0:
        t0 = time.time()
        om.step(emb[n + 1:n + 2], [cp])
        t += time.time() - t0
        n += 1
    om.free_cache(cp)
    per_layer = max(t / n - t_head, 1e-9) / nL
    return {"value": round(1.0 / (per_layer * cfg["n_layers"]), 3), "unit": "tok/s", **cpu_fields(threads()), "kind": "port",
            "sample": "oracle, %d of %d layers, the prompt's first %d tokens one at a time (%.1f s), head time taken out, per-layer cost scaled to %d layers"
                      % (nL, cfg["n_layers"], n, t, cfg["n_layers"])}
