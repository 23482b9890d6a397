"""The north-star logit bar, un-widened, where the reference arithmetic's chaos cannot compound: one decoder layer (plus the final
norm and the LM head) at the layer shapes of the BASELINE configurations, fed the same hidden-state rows and the same uploaded
KV on both sides. Bar: max-abs <= 2e-2 and <= 1e-2 of the row's largest |logit| (tests/models.py logits_close with floor 0).
The GEMMs are integer-exact up to the order of their f32 fold (1e-6 of the f64 sum; the oracle's single accumulator sits 2e-6 from
it), the attention is f32 against the oracle's f64 (held to 1e-4, about 1e-5 in practice). At the Qwen2-0.5B layer shape, and
wherever the residual stream dominates what the layer adds, the bar holds as stated. At the Llama-3-8B and Qwen3-MoE layer
shapes with a small residual stream it does not, for the GPU or for the oracle against itself: the oracle's own logits move by
more than four bars when its input changes by 1e-6, because the next per-32 quantizer turns a 1e-6 difference into flipped
codes. There the GPU is held beside that movement (it stays below it) and the share of logits beyond the stated bar is bounded.

Deeper models are compared under a bar widened by the oracle's own sensitivity (tests/test_gpu_model.py,
tests/test_gpu_baseline_shapes.py): per-32 int8 activation quantization at every matmul input amplifies a 1e-6 input change
into a change of a few 1e-2 in the logits within a few layers (tests/test_oracle_sensitivity.py). Here one layer is what
separates input and output, and the GPU must sit inside the bar as stated. The deep tests at the end hold the full-depth
Llama-3-8B-shape step and an 8-layer Qwen3-MoE-shape step to the widened bar and report how the deviation compares with the
oracle's own movement."""
import numpy as np
import pytest

from goinfer_amd import capi, synth, workloads
from oracle import binding as ob
from tests.models import Pair, dense_cfg, logits_close, near_tie_ok, perturbed

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = capi.Device(0)
    yield d
    d.close()


def one_step(pair, lens, hidden_sigma, seed, floor_eps=0.0):
    """Synthetic KV into both sides, then one batched step on hidden-state rows ~ N(0, hidden_sigma). Returns (gpu logits, oracle
    logits, oracle logits under a relative input perturbation of floor_eps or None)."""
    cfg, B = pair.cfg, len(lens)
    kvd, H = cfg["n_kv"] * cfg["head_dim"], cfg["hidden"]
    cap = int(max(lens)) + 2
    caches = [pair.oracle.new_cache(cap) for _ in range(B)]
    caches2 = [pair.oracle.new_cache(cap) for _ in range(B)] if floor_eps else None
    mx = int(max(lens))
    for l in range(cfg["n_layers"]):
        k = synth.normal(seed * 100 + 2 * l, mx * kvd, 1.0).reshape(mx, kvd)
        v = synth.normal(seed * 100 + 2 * l + 1, mx * kvd, 1.0).reshape(mx, kvd)
        for i, n in enumerate(lens):
            pair.gpu.kv_upload(i, l, 0, k[:n], v[:n])
            pair.oracle.cache_upload(caches[i], l, 0, k[:n], v[:n])
            if caches2:
                pair.oracle.cache_upload(caches2[i], l, 0, k[:n], v[:n])
    emb = synth.normal(seed * 7 + 3, B * H, hidden_sigma).reshape(B, H)
    pos = [int(n) for n in lens]
    moe = cfg.get("n_experts", 0) > 0
    o2 = None
    if moe:
        o, tr, wt = pair.oracle.step(emb, caches, want_weights=True)
        if caches2:
            o2 = pair.oracle.step(perturbed(emb, floor_eps, (seed, 0)), caches2, replay=(tr, wt))
        pair.gpu.moe_replay(tr, wt)  # the oracle's routing: a flipped expert is a different function (decoder/mlp.go moeSelOverride)
    else:
        o = pair.oracle.step(emb, caches)
        if caches2:
            o2 = pair.oracle.step(perturbed(emb, floor_eps, (seed, 0)), caches2)
    g, gid = pair.gpu.step_batch(list(range(B)), pos, emb, capi.WANT_LOGITS | capi.WANT_ARGMAX)
    for c in caches + (caches2 or []):
        pair.oracle.free_cache(c)
    return g, o, o2, gid


def hold_unwidened(g, o, what):
    """Every row inside the bar as stated: max-abs 2e-2 and 1e-2 of the row's largest |logit|. Returns the worst deviation in bars."""
    worst, beyond, n = measure(g, o)
    print("%s: worst deviation %.3f of the bar, %d of %d logits beyond it" % (what, worst, beyond, n))
    for b in range(len(o)):
        ok, d = logits_close(g[b], o[b], 0.0)
        assert ok, (what, b, d)
    return worst


def measure(g, o):
    worst, beyond, n = 0.0, 0, 0
    for b in range(len(o)):
        tol = min(2e-2, 1e-2 * float(np.abs(o[b]).max()))
        d = np.abs(g[b].astype(np.float64) - o[b].astype(np.float64))
        worst = max(worst, float(d.max()) / tol)
        beyond += int((d > tol).sum())
        n += d.size
    return worst, beyond, n


def hold_beside_the_oracles_own_movement(g, o, o2, what):
    """Where one layer already amplifies the attention's f32-against-f64 difference (about 1e-5 of its output) past the bar, the GPU
    is held to twice what the oracle itself moves by when its input changes by 1e-6, and to at most 2 % of the logits beyond the
    stated bar; both figures are printed."""
    floor = float(np.abs(o.astype(np.float64) - o2).max())
    worst, beyond, n = measure(g, o)
    w2, b2, _ = measure(o2, o)
    print("%s: GPU worst %.3f of the bar, %d of %d logits beyond it; the oracle under a 1e-6 input change: worst %.3f, %d beyond" % (what, worst, beyond, n, w2, b2))
    for b in range(len(o)):
        ok, d = logits_close(g[b], o[b], floor)
        assert ok, (what, b, d, floor)
    assert beyond <= 0.02 * n, (what, beyond, n)


def test_one_layer_llama3_8b_shape_short_contexts(dev):
    """With one to eight keys per sequence the attention is all but exact (one key: the stored value itself), and the layer still
    sits as far from the oracle as with thousands of keys: what is left is the order of the GEMMs' f32 folds. The kernels cut K over
    waves and fold the parts, the oracle runs one accumulator down all of K; the two differ by 2e-6 of the output's rms, the size
    of the oracle's own distance from the f64 sum, and the next per-32 quantizer turns that into flipped codes."""
    cfg = dict(workloads.llama3_8b_cfg(1), kv_f16=1)
    lens = np.random.default_rng(10).integers(1, 9, 32)
    for hidden_sigma in (0.02, 30.0):
        pair = Pair(cfg, seed=51, dev=dev, slots=32, ctx_cap=16)
        try:
            g, o, o2, gid = one_step(pair, lens, hidden_sigma, seed=60, floor_eps=1e-6)
            what = "llama3-8b layer, 1 to 8 keys, hidden sigma %g" % hidden_sigma
            if hidden_sigma >= 30.0:
                hold_unwidened(g, o, what)
            else:
                hold_beside_the_oracles_own_movement(g, o, o2, what)
        finally:
            pair.close()


@pytest.mark.parametrize("hidden_sigma", [0.02, 1.0, 10.0, 30.0])
def test_one_layer_llama3_8b_shape(dev, hidden_sigma):
    """hidden_sigma: the scale of the residual stream entering the layer (an embedding row, a mid-stack row, a late row). The smaller
    it is, the more of the layer's output is the attention's, whose f32 arithmetic differs from the oracle's f64 by about 1e-5."""
    cfg = dict(workloads.llama3_8b_cfg(1), kv_f16=1)
    lens = np.random.default_rng(11).integers(512, 4097, 32)
    pair = Pair(cfg, seed=51, dev=dev, slots=32, ctx_cap=int(lens.max()) + 8)
    try:
        g, o, o2, gid = one_step(pair, lens, hidden_sigma, seed=61, floor_eps=1e-6)
        what = "llama3-8b layer, contexts U[512,4096], hidden sigma %g" % hidden_sigma
        if hidden_sigma >= 10.0:
            hold_unwidened(g, o, what)
        else:
            hold_beside_the_oracles_own_movement(g, o, o2, what)
        for b in range(len(o)):
            assert near_tie_ok(o[b], int(gid[b]))
    finally:
        pair.close()


@pytest.mark.parametrize("hidden_sigma", [0.02, 1.0])
def test_one_layer_qwen2_05b_shape(dev, hidden_sigma):
    cfg = dense_cfg(n_layers=1, hidden=896, n_heads=14, n_kv=2, head_dim=64, inter=4864, vocab=151936, theta=1e6, eps=1e-6)
    lens = [17, 64, 128, 200]
    pair = Pair(cfg, seed=52, dev=dev, slots=4, ctx_cap=256)
    try:
        g, o, _, _ = one_step(pair, lens, hidden_sigma, seed=62)
        hold_unwidened(g, o, "qwen2-0.5b layer, hidden sigma %g" % hidden_sigma)
    finally:
        pair.close()


@pytest.mark.parametrize("hidden_sigma", [0.02, 1.0])
def test_one_layer_qwen3_moe_shape(dev, hidden_sigma):
    """On the oracle's routing (rd_moe_replay): every row is held to the bar, none is excused."""
    cfg = dict(workloads.qwen3_moe_cfg(1), kv_f16=1)
    lens = np.random.default_rng(12).integers(256, 2049, 16)
    pair = Pair(cfg, seed=53, dev=dev, slots=16, ctx_cap=int(lens.max()) + 8)
    try:
        g, o, o2, _ = one_step(pair, lens, hidden_sigma, seed=63, floor_eps=1e-6)
        what = "qwen3-moe layer, hidden sigma %g" % hidden_sigma
        if hidden_sigma >= 1.0:
            hold_unwidened(g, o, what)
        else:
            hold_beside_the_oracles_own_movement(g, o, o2, what)
    finally:
        pair.close()


def deep_step(dev, cfg, lens, seed, what):
    """One step through a deep stack under the widened bar, with the deviation set beside the oracle's own movement under input
    perturbation of 1e-6 (a few f32 ulps)."""
    pair = Pair(cfg, seed=seed, dev=dev, slots=len(lens), ctx_cap=int(max(lens)) + 8)
    try:
        g, o, o2, gid = one_step(pair, lens, 0.02, seed=seed + 10, floor_eps=1e-6)
        floor = float(np.abs(o - o2).max())
        dev_max = float(np.abs(g.astype(np.float64) - o).max())
        print("%s: GPU deviation %.4f, oracle movement under a 1e-6 input change %.4f" % (what, dev_max, floor))
        for b in range(len(o)):
            ok, d = logits_close(g[b], o[b], floor)
            assert ok, (what, b, d, floor)
            assert near_tie_ok(o[b], int(gid[b])), (what, "greedy token", b)
    finally:
        pair.close()


def test_full_depth_llama3_8b_shape_step(dev):
    """All 32 layers, B = 32, against the oracle (contexts kept to U[64,512] so the oracle's f32 caches stay small)."""
    cfg = dict(workloads.llama3_8b_cfg(32), kv_f16=1)
    lens = np.random.default_rng(13).integers(64, 513, 32)
    deep_step(dev, cfg, lens, 71, "llama3-8b shape, 32 layers")


def test_eight_layer_qwen3_moe_shape_step(dev):
    cfg = dict(workloads.qwen3_moe_cfg(8), kv_f16=1)
    lens = np.random.default_rng(14).integers(64, 513, 16)
    deep_step(dev, cfg, lens, 72, "qwen3-moe shape, 8 layers")
