"""What size of mistake do the un-widened single-layer parity tests catch?

tests/test_gpu_single_layer.py holds the GPU to the north-star bar as stated (max-abs 2e-2, 1e-2 of the row's largest |logit|) for one
decoder layer + final norm + head at the BASELINE layer shapes. A bar only pins an implementation if a plausible mistake breaks it.
Here the oracle is run against a deliberately wrong copy of itself (oracle.h OR_FAULT_*: RoPE rotated for the next position, a query
head reading its neighbour's kv head, a Q4_K sub-block scale taken from the neighbouring sub-block, the -dmin*m term dropped, the
row not seeing its own key, the attention softcap dropped, an int4 group scale taken from the next group) on the same set-ups, with
fewer rows so that it runs on a CPU in seconds, and the deviation is measured in bars. Every fault must land beyond one bar in every
set-up the GPU tests use un-widened: then a GPU kernel with that fault fails there too. The measured factors are printed.
The set-up with the late-layer residual stream (sigma 30) is the weakest by construction (the layer's own contribution
is a few per cent of the stream), which is why its numbers matter most."""
import numpy as np
import pytest

from goinfer_amd import synth, workloads
from oracle import binding as ob
from tests.models import Pair, dense_cfg


def bars(got, want):
    worst = 0.0
    for b in range(len(want)):
        tol = min(2e-2, 1e-2 * float(np.abs(want[b]).max()))
        worst = max(worst, float(np.abs(got[b].astype(np.float64) - want[b].astype(np.float64)).max()) / tol)
    return worst


def oracle_layer(pair, lens, hidden_sigma, seed, fault, replay=None):
    """One step of the oracle's layer on hidden-state rows ~ N(0, sigma) over synthetic KV (the set-up of test_gpu_single_layer.one_step)."""
    cfg, B = pair.cfg, len(lens)
    kvd, H = cfg["n_kv"] * cfg["head_dim"], cfg["hidden"]
    mx = int(max(lens))
    caches = [pair.oracle.new_cache(mx + 2) for _ in range(B)]
    for l in range(cfg["n_layers"]):
        k = synth.normal(seed * 100 + 2 * l, mx * kvd, 1.0).reshape(mx, kvd)
        v = synth.normal(seed * 100 + 2 * l + 1, mx * kvd, 1.0).reshape(mx, kvd)
        for i, n in enumerate(lens):
            pair.oracle.cache_upload(caches[i], l, 0, k[:n], v[:n])
    emb = synth.normal(seed * 7 + 3, B * H, hidden_sigma).reshape(B, H)
    ob.set_fault(fault)
    try:
        if cfg.get("n_experts", 0) > 0:
            if replay is None:
                out = pair.oracle.step(emb, caches, want_weights=True)
            else:
                out = (pair.oracle.step(emb, caches, replay=replay),)
        else:
            out = (pair.oracle.step(emb, caches),)
    finally:
        ob.set_fault("none")
        for c in caches:
            pair.oracle.free_cache(c)
    return out


DENSE_FAULTS = ["rope_pos", "gqa_head", "q4k_scale_index", "q4k_no_min", "causal_range"]

SETUPS = {
    # name: (cfg, lens, sigmas the GPU test holds un-widened)
    "qwen2-0.5b layer": (dense_cfg(n_layers=1, hidden=896, n_heads=14, n_kv=2, head_dim=64, inter=4864, vocab=151936, theta=1e6, eps=1e-6),
                         [17, 64, 128, 200], (0.02, 1.0)),
    "llama3-8b layer": (dict(workloads.llama3_8b_cfg(1), kv_f16=1), [int(n) for n in np.random.default_rng(11).integers(512, 4097, 4)], (10.0, 30.0)),
}


@pytest.mark.parametrize("name", sorted(SETUPS))
def test_dense_layer_faults_land_beyond_the_bar(name):
    cfg, lens, sigmas = SETUPS[name]
    pair = Pair(cfg, seed=51, dev=None)
    ob.set_threads(8)
    for sigma in sigmas:
        (want,) = oracle_layer(pair, lens, sigma, 61, "none")
        (again,) = oracle_layer(pair, lens, sigma, 61, "none")
        assert np.array_equal(want, again)  # the knob leaves the faithful oracle alone
        for fault in DENSE_FAULTS:
            (got,) = oracle_layer(pair, lens, sigma, 61, fault)
            b = bars(got, want)
            print("%s, hidden sigma %g, fault %s: %.1f bars" % (name, sigma, fault, b))
            assert b > 1.0, (name, sigma, fault, b)


SOFTCAP_THAT_BITES = 0.1  # random-init scores are ~0.1: Gemma's 50 would never bend them, and a dropped cap would go unseen


def test_softcap_fault_lands_beyond_the_bar():
    """tests/test_gpu_model.py::test_softcap_model runs this cap; with a cap of 50 on the same model the fault stays under one bar,
    i.e. such a test could not tell whether the kernels apply a softcap at all."""
    lens = [4, 70, 200]
    seen = {}
    for cap in (SOFTCAP_THAT_BITES, 50.0):
        pair = Pair(dense_cfg(n_layers=2, softcap=cap), seed=4, dev=None)
        (want,) = oracle_layer(pair, lens, 0.02, 62, "none")
        (got,) = oracle_layer(pair, lens, 0.02, 62, "no_softcap")
        seen[cap] = bars(got, want)
        print("two-layer model, softcap %g, fault no_softcap: %.4f bars" % (cap, seen[cap]))
    assert seen[SOFTCAP_THAT_BITES] > 1.0 and seen[50.0] < 1.0


def test_moe_layer_faults_land_beyond_the_bar():
    """The Qwen3-MoE layer shape at hidden sigma 1 on a replayed routing (what test_one_layer_qwen3_moe_shape holds un-widened)."""
    cfg = dict(workloads.qwen3_moe_cfg(1), kv_f16=1)
    lens = [int(n) for n in np.random.default_rng(12).integers(256, 2049, 4)]
    pair = Pair(cfg, seed=53, dev=None)
    ob.set_threads(8)
    want, tr, wt = oracle_layer(pair, lens, 1.0, 63, "none")
    for fault in ["rope_pos", "gqa_head", "q4k_scale_index", "causal_range", "w4a8_scale_index"]:
        (got,) = oracle_layer(pair, lens, 1.0, 63, fault, replay=(tr, wt))
        b = bars(got, want)
        print("qwen3-moe layer, hidden sigma 1, fault %s: %.1f bars" % (fault, b))
        assert b > 1.0, (fault, b)
