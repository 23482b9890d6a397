#!/usr/bin/env python3
"""Benchmark of the ragged batched decode step on one MI355X.

A step is one pass of the hot path over one batch: the greedy decode step of 32 ragged sequences of a Llama-3-8B-shaped
Q4_K model (BASELINE.json configs[3], the configuration its metric is quoted on). Inputs (weights, KV caches, embedding
table) are resident in HBM before the timed region; the greedy chain runs on the device (argmax -> embedding gather).
Prints ONE JSON line with the whole-job tok/s, the roofline of the dominant kernel and a CPU baseline (the oracle's
restatement of goinfer's CPU path, timed on this box's host cores on a bounded sample of the same workload).

--workload c2 | c3 | c5 runs the other measurement configurations BASELINE.json names instead (the Q4_K GEMM microbench, the
ragged attention microbench, the Qwen3-MoE-shaped step; kquant: the Q5_K / Q6_K GEMMs beside Q4_K), topk (the device-side top-K of logits rows) or prefill (a 2048-token prompt
pass into the same paged KV) and prints one line of the same form for that workload.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

from bench_micro import counter_traffic, cpu_fields  # noqa: E402

HBM_PEAK_GBS = 8000.0
CPU_LAYERS = 8       # layers of the model the CPU baseline runs
CPU_SECONDS = 12.0   # about this much timed CPU work
CPU_MAX_STEPS = 64


def log(msg):
    print("[bench %6.1fs] %s" % (time.time() - T0, msg), file=sys.stderr, flush=True)


def cpu_baseline(res, cfg, lens, kept_kv, threads, kv="f16"):
    """The oracle's decodeMultiStep on the first layers of the same model, the same 32 ragged sequences and KV, greedy
    steps for about ten seconds; the per-layer cost scaled to the full depth. Returns (tok/s, description of the sample)."""
    from oracle import binding as ob
    ob.set_threads(threads)
    nL = len(res.kept)
    layers = []
    for kp in res.kept:
        lw = {p: ob.WMat(ob.OR_Q4K, kp[p][1], kp[p][2], kp[p][0], act_group=32) for p in ("q", "k", "v", "o", "gate", "up", "down")}
        lw["attn_norm"], lw["ffn_norm"] = kp["attn_norm"], kp["ffn_norm"]
        layers.append(lw)
    c = dict(cfg)
    c.update(n_layers=nL, kv_f16=1 if kv == "f16" else 2)
    hq, hs = res.head
    head = ob.WMat(ob.OR_W8A8, hq.shape[0], hq.shape[1], hq, hs, act_group=32)
    from goinfer_amd.workloads import inv_freq
    om = ob.OracleModel(c, layers, res.final_norm, head, inv_freq(cfg["head_dim"], cfg["theta"]))
    B = len(lens)
    caches = []
    for i, n in enumerate(lens):
        cp = om.new_cache(int(n) + CPU_MAX_STEPS + 2)
        for l in range(nL):
            k, v = kept_kv[l]
            om.cache_upload(cp, l, 0, k[:n], v[:n])  # UploadKV: narrowed to f16 as the cache stores it
        caches.append(cp)
    ids = np.arange(B) * 977 % cfg["vocab"]
    emb = res.embed_rows(ids)
    om.step(emb, caches)  # untimed: page in the weights
    n_steps, t_step = 0, 0.0
    while n_steps < CPU_MAX_STEPS - 1 and t_step < CPU_SECONDS:
        t0 = time.time()
        logits = om.step(emb, caches)
        t_step += time.time() - t0
        n_steps += 1
        emb = res.embed_rows(np.array([ob.argmax(r) for r in logits]))
    # the head alone, to separate it from the per-layer cost
    t0 = time.time()
    for _ in range(3):
        ob.matmul(head, emb)
    t_head = (time.time() - t0) / 3
    t_total, t_step = t_step, t_step / n_steps
    for cp in caches:
        om.free_cache(cp)
    per_layer = max(t_step - t_head, 1e-9) / nL
    full = per_layer * cfg["n_layers"] + t_head
    sample = ("oracle decodeMultiStep, %d of %d layers + int8 head, B=%d at the run's context lengths, %d greedy steps (%.1f s), "
              "per-layer cost scaled to %d layers" % (nL, cfg["n_layers"], B, n_steps, t_total, cfg["n_layers"]))
    return B / full, sample


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=32, help="model depth (32 = the Llama-3-8B shape; fewer only for debugging)")
    ap.add_argument("--batch", type=int, default=32)
    ap.add_argument("--seed", type=int, default=1234)
    ap.add_argument("--ctx-min", type=int, default=512, help="c4: shortest context (the configuration's own range is 512..4096)")
    ap.add_argument("--ctx-max", type=int, default=4096, help="c4: longest context")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--kv", default="f16", choices=["f16", "i8"],
                    help="KV cache element (c4 and c3): f16 as the metric is quoted, or goinfer's int8 cache (KVQuant i8), a variant of the workload")
    ap.add_argument("--exp-act-group", type=int, default=0, choices=[0, 32],
                    help="c5: the experts' activation quantization, 0 = one int8 scale per token row (the configuration as stated), 32 = per group of 32 (a variant)")
    ap.add_argument("--m", type=int, default=0, help="c2: only this batch width (for counter runs: one shape per kernel name)")
    ap.add_argument("--workload", default="c4", choices=["c4", "c2", "c3", "c5", "kquant", "topk", "prefill", "issue"],
                    help="c4 (default): the Llama-3-8B-shape step the metric is quoted on; c2: Q4_K GEMM microbench; c3: ragged "
                         "attention microbench; c5: Qwen3-MoE-shape step; kquant: Q4_K / Q5_K / Q6_K GEMMs at the FFN and head shapes; topk: "
                         "the device-side top-K of logits rows; prefill: a 2048-token prompt pass into the same paged KV; issue: what a SIMD sustains "
                         "of the int8 GEMMs' inner-loop instruction mix (no memory)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this backend is single-GPU (goinfer has no collective path); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    return args


def run_c4(args):

    from goinfer_amd import capi, workloads

    cfg = workloads.llama3_8b_cfg(args.layers)
    B = args.batch
    rng = np.random.default_rng(args.seed)
    lens = rng.integers(args.ctx_min, args.ctx_max + 1, B).astype(np.int64)  # context lengths uniform in [512, 4096] unless asked otherwise
    ids0 = rng.integers(0, cfg["vocab"], B).astype(np.int32)
    cap = int(lens.max()) + args.steps + args.warmup + 48  # the timed steps, then the profiling and enqueue-cost steps after them
    dev = capi.Device(0)
    log("building %s, %d layers" % (cfg["name"], cfg["n_layers"]))
    res = workloads.Resident(dev, cfg, seed=args.seed, slots=B, ctx_cap=cap, keep_layers=0 if args.no_cpu else min(CPU_LAYERS, args.layers), progress=log, kv=args.kv)
    kept_kv = res.prefill_kv(lens, progress=log)
    slots = np.arange(B, dtype=np.int32)

    # ---- timed region: K greedy decode steps after W warmup steps, HIP events per step on the launch stream ----
    dev.sync()
    t0 = time.time()
    ms = res.model.bench_steps(slots, lens, ids0, args.warmup, args.steps)
    dev.sync()
    wall = time.time() - t0
    total_ms = float(ms.sum())
    tok_s = B * args.steps / (total_ms / 1e3)
    log("steps: %.3f ms mean, %.3f ms median; wall for warmup+steps %.2f s" % (ms.mean(), float(np.median(ms)), wall))

    # ---- algorithmic bytes of a step at the mid-run context lengths ----
    mid = lens + args.warmup + args.steps // 2
    kv_pos_bytes = workloads.kv_bytes_per_position(cfg, args.kv)
    kv_read = float((mid + 1).sum()) * kv_pos_bytes
    w_bytes = workloads.weight_bytes(cfg)
    step_bytes = w_bytes + kv_read + B * kv_pos_bytes
    step_gbs = step_bytes / (ms.mean() / 1e3) / 1e9

    # ---- roofline of the dominant kernel: the ragged flash-decode attention (KV is ~70 % of the step's bytes) ----
    pos_prof = (lens + args.warmup + args.steps).astype(np.int32)
    prof = {}
    for rep in range(3):
        p = res.model.bench_profile(slots, pos_prof + rep, ids0)
        for k, (t, n) in p.items():
            a = prof.setdefault(k, [0.0, 0])
            a[0] += t
            a[1] += n
    kern = "attn_partial"
    single_ms = prof[kern][0] / prof[kern][1]  # an event pair around every launch: carries the events' own 2-3 us
    # every layer's launch back to back between one pair of events: the kernel with its work list, tables and q still in L2
    chain = [res.model.bench_attn_chain(slots, pos_prof + rep, ids0) for rep in range(3)]
    chain_ms = float(np.mean([c[0] for c in chain]))
    # the kernel's average launch duration where it runs: whole steps against the same steps without their attention launches,
    # each step between its own pair of events. This is the figure the profiler's kernel duration agrees with.
    avg_ms, _ = res.model.bench_attn_in_step(slots, pos_prof + 2, ids0, 24)
    kernel_name = res.model.attn_kernel_name()  # the variant this work list takes (wide blocks, two units in flight, int8 cache)
    # per launch (one layer): every sequence's K and V rows once (f16, or int8 and their scales), plus q in and partial results out
    G = cfg["n_heads"] // cfg["n_kv"]
    kv_launch = float((pos_prof + 2).sum()) * kv_pos_bytes / cfg["n_layers"]
    q_launch = B * cfg["n_heads"] * cfg["head_dim"] * 4
    achieved = (kv_launch + q_launch) / (avg_ms / 1e3) / 1e9
    traffic, t_ratio, t_src = counter_traffic("%s/%s/%s" % (kern, cfg["name"], args.kv), kv_launch + q_launch)
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": traffic, "traffic_ratio": t_ratio, "traffic_source": t_src,
                "kernel": kernel_name, "avg_launch_ms": round(avg_ms, 5),
                "avg_launch_ms_event_pair_per_launch": round(single_ms, 5),
                "avg_launch_ms_back_to_back": round(chain_ms, 5),
                "timing": "HIP events on the launch stream around whole steps at the context lengths right after the timed ones: (a step - the same step "
                          "without its attention launches) / layers, the median of 24 pairs of steps; agrees with rocprofv3's kernel duration. The same kernel launched "
                          "back to back for all layers between one pair of events (its work list, tables and q then stay in L2) reads about 2 us less "
                          "(avg_launch_ms_back_to_back); an event pair around every single launch about 2 us more (avg_launch_ms_event_pair_per_launch)",
                "algorithmic_bytes_per_launch": int(kv_launch + q_launch),
                "step_frac": round(step_gbs / HBM_PEAK_GBS, 4)}
    classes = {k: {"ms_per_step": round(v[0] / 3, 4), "launches_per_step": v[1] // 3} for k, v in prof.items()}

    # ---- the host's cost of enqueueing a step: the captured graph's one launch against the eager launches ----
    host_us = {}
    at = pos_prof + 3  # where the profiling passes left the slots
    for mode, on in (("graph", True), ("eager", False)):
        if not res.model.set_graph(on):  # declined under a profiler: the eager figure only
            host_us[mode] = None
            continue
        # each call takes 3 settling steps and 4 timed ones (the depth of the step's staging ring: a fifth would wait for the GPU)
        runs = []
        for _ in range(3):
            runs.append(res.model.bench_enqueue(slots, at.astype(np.int32), ids0, 4))
            at = at + 7
        host_us[mode] = round(float(np.median(runs)), 1)
    res.model.set_graph(True)
    captures, replays = res.model.graph_stats()

    # ---- a plain copy kernel of known size: the practical HBM rate, and the yardstick the traffic counters are scaled by ----
    COPY_BYTES = 1 << 30
    cms = dev.bench_kernel("copy", [COPY_BYTES], 2, 6)
    copy_gbs = 2 * COPY_BYTES / (float(np.median(cms)) / 1e3) / 1e9

    cpu = None
    if not args.no_cpu:
        threads = min(16, len(os.sched_getaffinity(0)))
        log("CPU baseline on %d threads" % threads)
        v, sample = cpu_baseline(res, cfg, lens, kept_kv, threads, args.kv)
        cpu = dict({"value": round(v, 3), "unit": "tok/s"}, **cpu_fields(threads), kind="port", sample=sample)
    res.close()
    dev.close()

    out = {
        "metric": "batch-32 decode tok/s, Llama-3-8B-shape Q4_K; achieved HBM GB/s vs peak",
        "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(float(ms.mean()), 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic: N(0,0.02) weights quantized to Q4_K (int8 head), N(0,1) KV, random token ids",
        "config": {"workload": "configs[3]: %s, %d layers, B=%d ragged, ctx U[%d,%d], greedy decode%s"
                               % (cfg["name"], cfg["n_layers"], B, args.ctx_min, args.ctx_max, "" if args.kv == "f16" else " (variant: int8 KV cache)"), "kv": args.kv,
                   "batch": B, "ctx_min": int(lens.min()), "ctx_max": int(lens.max()), "ctx_mean": float(lens.mean()), "seed": args.seed},
        "step_hbm": {"algorithmic_bytes_per_step": int(step_bytes), "achieved_GBs": round(step_gbs, 1), "frac_of_peak": round(step_gbs / HBM_PEAK_GBS, 4),
                     "weights_bytes": int(w_bytes), "kv_read_bytes": int(kv_read)},
        "roofline": roofline,
        "copy_kernel": {"bytes_read": COPY_BYTES, "bytes_written": COPY_BYTES, "GBs": round(copy_gbs, 1)},
        "kernel_classes": classes,
        "host_enqueue_us_per_step": dict(host_us, note="wall clock of the host loop that enqueues a step, GPU not waited for; the timed steps above replay the graph"),
        "graph": {"captures": captures, "steps_replayed": replays},
        "cpu_baseline": cpu,
    }
    print(json.dumps(out, default=float))


if __name__ == "__main__":
    T0 = time.time()
    _args = parse_args()
    if _args.workload == "c4":
        run_c4(_args)
    else:
        import bench_micro
        bench_micro.T0 = T0
        {"c2": bench_micro.run_c2, "c3": bench_micro.run_c3, "c5": bench_micro.run_c5, "kquant": bench_micro.run_kquant,
         "topk": bench_micro.run_topk, "prefill": bench_micro.run_prefill, "issue": bench_micro.run_issue}[_args.workload](_args)
