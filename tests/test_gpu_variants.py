"""The knobs of the decode path that are not on the five benchmark configurations: router variants (sigmoid scoring, selection
bias, group-limited selection, routed scaling factor; decoder/mlp.go:130-228), attention sinks and the sliding window
(decoder/attention.go:57-143, 305-322; kvmgr.WindowNeedStart). Kernel level against the oracle (routing bit for bit, attention to
the flash-decode bar of 1e-4), then whole models through the step."""
import numpy as np
import pytest

from goinfer_amd import capi, synth
from oracle import binding as ob
from tests.models import Pair, dense_cfg, moe_cfg
from tests.test_gpu_attention import i8_round_trip
from tests.test_gpu_model import check

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = capi.Device(0)
    yield d
    d.close()


@pytest.mark.parametrize("nE,k,sigmoid,use_bias,n_group,topk_group,scale,norm", [
    (128, 8, True, True, 8, 4, 2.5, True),      # DeepSeek-V3 style: sigmoid + bias + groups + scale
    (64, 6, True, True, 0, 0, 1.0, True),       # GLM: sigmoid + bias
    (128, 8, False, True, 0, 0, 0.0, True),     # softmax with a selection bias
    (160, 4, True, False, 4, 2, 16.0, False),   # groups without a bias
    (30, 4, True, True, 4, 1, 0.0, True),       # experts past the last whole group are never eligible
    (8, 6, True, True, 4, 1, 0.0, True),        # fewer eligible experts than k: the row comes back short
    (256, 8, False, False, 0, 0, 0.0, True),    # the plain softmax router at the widest row
])
def test_route_variants_bit_exact(dev, nE, k, sigmoid, use_bias, n_group, topk_group, scale, norm):
    rng = np.random.default_rng(nE * 7 + k)
    T = 16
    logits = (rng.standard_normal((T, nE)) * 2).astype(np.float32)
    logits[3] = np.round(logits[3])          # ties
    logits[4] = 0.0                          # all equal: the lowest indices win
    bias = (rng.standard_normal(nE) * 0.3).astype(np.float32) if use_bias else None
    idx, wgt = dev.moe_route(logits, k, norm, bias=bias, sigmoid=sigmoid, scale=scale, n_group=n_group, topk_group=topk_group)
    for t in range(T):
        wi, ww = ob.route_experts(logits[t], k, norm, scale, bias=bias, sigmoid=sigmoid, n_group=n_group, topk_group=topk_group)
        n = len(wi)
        assert np.array_equal(idx[t, :n], wi), (t, idx[t], wi)
        assert np.array_equal(wgt[t, :n].view(np.uint32), ww.view(np.uint32)), (t, wgt[t], ww)


@pytest.mark.parametrize("kv", ["f16", "i8"])
@pytest.mark.parametrize("hd,nH,nKV", [(128, 8, 2), (64, 8, 8)])
def test_attention_window_and_sinks(dev, kv, hd, nH, nKV):
    """Rows over windowed contexts, with and without sinks and softcap, against the oracle's f64 attention over the rows as the
    cache holds them; and a row in a ragged batch equals the row alone, bit for bit."""
    lens = [1, 5, 63, 64, 65, 130, 700, 2000]
    kvd = nKV * hd
    ks = [synth.normal(100 + i, n * kvd).reshape(n, kvd) for i, n in enumerate(lens)]
    vs = [synth.normal(200 + i, n * kvd).reshape(n, kvd) for i, n in enumerate(lens)]
    q = synth.normal(9, len(lens) * nH * hd).reshape(len(lens), nH * hd)
    sinks = synth.normal(11, nH, 2.0)
    scale = hd ** -0.5
    hold = (lambda x: ob.f16_round_trip(x)) if kv == "f16" else (lambda x: i8_round_trip(x, nKV, hd))
    for window, sk, cap in ((0, sinks, 0.0), (48, None, 0.0), (100, sinks, 30.0), (1, sinks, 0.0), (4096, None, 0.0)):
        got = dev.attn_ragged_ex(lens, np.concatenate(ks), np.concatenate(vs), q, nH, nKV, hd, scale, cap, kv=kv, window=window, sinks=sk)
        for i, n in enumerate(lens):
            start = max(n - window, 0) if window else 0
            want = ob.attend(q[i], hold(ks[i]), hold(vs[i]), n, nH, nKV, hd, scale, cap, start=start, sinks=sk)
            assert np.abs(got[i] - want).max() <= 1e-4 * max(1.0, np.abs(want).max()), (window, i, n)
        solo = dev.attn_ragged_ex(lens[6:7], ks[6], vs[6], q[6:7], nH, nKV, hd, scale, cap, kv=kv, window=window, sinks=sk)
        assert np.array_equal(solo[0].view(np.uint32), got[6].view(np.uint32))


def test_attention_window_rows_of_one_sequence(dev):
    """Several consecutive positions of a sequence in one call (a prompt pass), each row with its own window start: equal to the
    rows computed one by one, bit for bit, and to the oracle."""
    nH, nKV, hd, n, nq, window = 8, 2, 128, 300, 7, 70
    kvd = nKV * hd
    k, v = synth.normal(1, n * kvd).reshape(n, kvd), synth.normal(2, n * kvd).reshape(n, kvd)
    q = synth.normal(3, nq * nH * hd).reshape(nq, nH * hd)
    scale = hd ** -0.5
    got = dev.attn_ragged_ex([n], k, v, q, nH, nKV, hd, scale, nq=[nq], window=window)
    for j in range(nq):
        ln = n - nq + 1 + j
        one = dev.attn_ragged_ex([ln], k[:ln], v[:ln], q[j:j + 1], nH, nKV, hd, scale, window=window)
        assert np.array_equal(one[0].view(np.uint32), got[j].view(np.uint32)), j
        want = ob.attend(q[j], ob.f16_round_trip(k), ob.f16_round_trip(v), ln, nH, nKV, hd, scale, start=max(ln - window, 0))
        assert np.abs(got[j] - want).max() <= 1e-4 * max(1.0, np.abs(want).max())


def test_model_with_window_and_sinks(dev):
    """A dense model whose even layers have a sliding window of 24 positions and whose every layer has attention sinks, through
    ragged prompts that outgrow the window, then batched greedy steps, against the oracle."""
    cfg = dict(dense_cfg(n_layers=4, hidden=256, n_heads=4, n_kv=2, head_dim=64, inter=512, vocab=512), window=24, attn_sinks=1)
    rng = np.random.default_rng(21)
    check(Pair(cfg, seed=31, dev=dev, slots=8), [list(rng.integers(0, 512, n)) for n in (3, 30, 70)], steps=4)
    # and the window is not ignored: the same model without it answers differently once a context has outgrown it
    a, b = Pair(cfg, seed=31, dev=dev, slots=2), Pair(dict(cfg, window=0), seed=31, dev=dev, slots=2)
    try:
        toks = list(rng.integers(0, 512, 40))
        for p, t in enumerate(toks):
            la, _ = a.gpu.step_batch([0], [p], a.emb[[t]])
            lb, _ = b.gpu.step_batch([0], [p], b.emb[[t]])
            if p < 24:
                assert np.array_equal(la.view(np.uint32), lb.view(np.uint32)), p  # inside the window the two are one model
        assert np.abs(la - lb).max() > 1e-3
    finally:
        a.close()
        b.close()


def test_moe_model_with_deepseek_style_router(dev):
    """Sigmoid scores, a selection bias per layer, group-limited selection (4 groups, the best 2), weights renormalized and scaled
    by 2.5, through the step against the oracle on the oracle's replayed routing: every row of every step is held to the bar, none
    excused; the GPU's own routing on its own hidden states is only counted."""
    from tests.test_gpu_model import run_moe_replayed
    cfg = dict(moe_cfg(n_layers=2, hidden=256, n_heads=4, n_kv=2, head_dim=64, n_experts=16, top_k=4, exp_inter=128, exp_act_group=0),
               router_sigmoid=1, router_bias=1, n_group=4, topk_group=2, router_scale=2.5)
    rng = np.random.default_rng(5)
    worst, floor, agree, total = run_moe_replayed(Pair(cfg, seed=41, dev=dev, slots=8), [list(rng.integers(0, 512, n)) for n in (2, 20)], steps=4)
    print("worst logit deviation %.4f, oracle noise floor %.4f, free-running expert index agreement %d/%d" % (worst, floor, agree, total))
    assert agree >= 0.9 * total, (agree, total)


GEMMA2 = dict(window=24, post_norms=1, norm_add_one=1, act_gelu_tanh=1, final_softcap=30.0)


@pytest.mark.parametrize("hidden,heads", [(256, 4), (384, 6)])
def test_gemma2_style_block(dev, hidden, heads):
    """Gemma 2's block through the step against the oracle (which reproduces the reference's gemma2-tiny golden): (1 + w) norms
    before and after both branches, GeGLU, attention softcap 50, a window on the even layers, final-logit softcap 30. hidden 256 runs
    the fused gate|up kernel, hidden 384 the int8-row lane with the separate activation kernel."""
    cfg = dict(dense_cfg(n_layers=4, hidden=hidden, n_heads=heads, n_kv=2, head_dim=64, inter=512, vocab=512, theta=1e4, eps=1e-6, softcap=50.0), **GEMMA2)
    cfg["attn_scale"] = 144.0 ** -0.5  # query_pre_attn_scalar, not head_dim
    rng = np.random.default_rng(61)
    check(Pair(cfg, seed=71, dev=dev, slots=8), [list(rng.integers(0, 512, n)) for n in (3, 30, 70)], steps=4)


def test_gemma2_knobs_are_not_ignored(dev):
    """Each knob of the block changes the GPU's answer: the same weights without it give different logits. (The (1 + w) scale is
    not in the list: the helper stores the same weights as deviations from one when it is on, so ignoring it on the GPU would
    scale every norm by about 0.02 and fail the comparison with the oracle above.)"""
    cfg = dict(dense_cfg(n_layers=2, hidden=256, n_heads=4, n_kv=2, head_dim=64, inter=512, vocab=512, softcap=50.0), **GEMMA2)
    cfg["final_softcap"] = 2.0
    toks = list(np.random.default_rng(62).integers(0, 512, 6))

    def last_logits(c):
        p = Pair(c, seed=72, dev=dev, slots=2)
        try:
            for pos, t in enumerate(toks):
                lg, _ = p.gpu.step_batch([0], [pos], p.emb[[t]] * np.float32(16.0))
            ref = p.oracle.new_cache(16)
            for t in toks:
                want = p.oracle.step(p.emb[[t]] * np.float32(16.0), [ref])
            p.oracle.free_cache(ref)
            assert np.abs(lg - want).max() <= 2e-2
            return lg
        finally:
            p.close()

    base = last_logits(cfg)
    assert np.abs(base).max() < 2.0  # capped
    for knob in ("post_norms", "act_gelu_tanh", "final_softcap"):
        assert np.abs(last_logits(dict(cfg, **{knob: 0})) - base).max() > 1e-3, knob


def test_gemma2_fused_gateup_equals_separate_kernels(dev, monkeypatch):
    """The gate|up kernel with GeGLU in its epilogue against the plain GEMM followed by the activation kernel: the same bits."""
    cfg = dict(dense_cfg(n_layers=2, hidden=256, n_heads=4, n_kv=2, head_dim=64, inter=512, vocab=512), **GEMMA2)
    rng = np.random.default_rng(63)
    toks = rng.integers(0, 512, (3, 40))
    outs = []
    for off in (False, True):
        if off:
            monkeypatch.setenv("ROCMDECODE_NO_FUSED_GATEUP", "1")
        p = Pair(cfg, seed=73, dev=dev, slots=40)
        try:
            got = [p.gpu.step_batch(list(range(40)), [pos] * 40, p.emb[toks[pos]])[0] for pos in range(3)]
            outs.append(np.stack(got))
        finally:
            p.close()
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))


def test_granite_style_multipliers(dev):
    """Granite's block is a llama block with three multipliers (decoder/arch_granite.go:50-62): the embedding's arrives with the
    rows, the attention scale is the model's, and the logits are divided by logits_scaling after the head."""
    cfg = dict(dense_cfg(n_layers=2, hidden=256, n_heads=4, n_kv=2, head_dim=64, inter=512, vocab=512), logit_scale=6.0)
    cfg["attn_scale"] = 0.0625
    rng = np.random.default_rng(64)
    check(Pair(cfg, seed=74, dev=dev, slots=4), [list(rng.integers(0, 512, n)) for n in (5, 40)], steps=3)
    a, b = Pair(cfg, seed=74, dev=dev, slots=2), Pair(dict(cfg, logit_scale=0.0), seed=74, dev=dev, slots=2)
    try:
        e = a.emb[[7]]
        la, _ = a.gpu.step_batch([0], [0], e)
        lb, _ = b.gpu.step_batch([0], [0], e)
        assert np.array_equal(la.view(np.uint32), (lb * np.float32(1.0 / 6.0)).view(np.uint32))  # one rounded multiply per logit
    finally:
        a.close()
        b.close()


def test_a_layer_set_back_to_no_window_no_longer_counts(dev):
    """rd_model_set_window(layer, 0) takes the layer's window back: the model's window is what its layers hold, so another length
    is then accepted, and two different lengths at once are still declined."""
    cfg = dense_cfg(n_layers=3)
    from tests.util import inv_freq
    m = capi.Model(dev, cfg, inv_freq(cfg["head_dim"], cfg["theta"]))
    try:
        m.set_window(0, 16)
        with pytest.raises(capi.RocmError, match="different lengths"):
            m.set_window(1, 8)
        m.set_window(0, 0)
        m.set_window(1, 8)
        m.set_window(2, 8)
        with pytest.raises(capi.RocmError, match="different lengths"):
            m.set_window(0, 16)
    finally:
        m.close()
