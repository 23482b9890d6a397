"""The ragged step and the prefill bridge (rd_step_ragged, rd_prefill_last) against the single-token path and the oracle.

goinfer's contract for StepRagged / ForwardN (resident/forward.go:9-16, resident/subsystems.go:112-117): row j of a sequence
equals that sequence's own Forward at Pos+j bit for bit, and the K/V a prefill pass leaves behind are those the token-by-token
path would have left. Both are asserted with array_equal; the oracle comparison carries the usual noise-floor bar."""
import numpy as np
import pytest

from goinfer_amd import capi
from oracle import binding as ob
from tests.models import Pair, dense_cfg, logits_close, moe_cfg, perturbed

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = capi.Device(0)
    yield d
    d.close()


def bits(x):
    return np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)


def forward_tokens(pair, slot, toks, start=0):
    """Token by token on one slot; returns every position's logits."""
    return np.stack([pair.gpu.forward(slot, start + p, pair.emb[t]) for p, t in enumerate(toks)])


@pytest.mark.parametrize("cfg", [dense_cfg(), moe_cfg()], ids=["dense", "moe"])
def test_ragged_rows_equal_single_token_steps(dev, cfg):
    pair = Pair(cfg, seed=51, dev=dev, slots=8, ctx_cap=256)
    rng = np.random.default_rng(5)
    a, b, c = (list(rng.integers(0, cfg["vocab"], n)) for n in (5, 1, 40))
    want = [forward_tokens(pair, 4 + i, t) for i, t in enumerate((a, b, c))]  # twins on slots 4..6
    # one call: 5 + 1 + 40 rows = two passes of the step; the 40-row sequence straddles them
    got, ids = pair.gpu.step_ragged([0, 1, 2], [0, 0, 0], [pair.emb[a], pair.emb[b], pair.emb[c]], capi.WANT_LOGITS | capi.WANT_ARGMAX)
    off = 0
    for w in want:
        assert np.array_equal(bits(got[off:off + len(w)]), bits(w))
        assert np.array_equal(ids[off:off + len(w)], np.argmax(w, axis=1))
        off += len(w)
    # the KV left behind is the token-by-token KV: the next single-token step agrees bit for bit
    nxt = int(rng.integers(0, cfg["vocab"]))
    for s, n in ((0, 5), (1, 1), (2, 40)):
        assert np.array_equal(bits(pair.gpu.forward(s, n, pair.emb[nxt])), bits(pair.gpu.forward(4 + s, n, pair.emb[nxt])))
    # a second ragged call continues where the first stopped (decode row + verify rows)
    more = list(rng.integers(0, cfg["vocab"], 3))
    g2, _ = pair.gpu.step_ragged([2, 0], [41, 6], [pair.emb[more], pair.emb[more[:1]]])
    w2 = forward_tokens(pair, 6, more, start=41)
    assert np.array_equal(bits(g2[:3]), bits(w2))
    pair.close()


def test_prefill_last_matches_token_by_token_and_oracle(dev):
    cfg = dense_cfg()
    pair = Pair(cfg, seed=52, dev=dev, slots=4, ctx_cap=256)
    rng = np.random.default_rng(6)
    toks = list(rng.integers(0, cfg["vocab"], 97))  # one pass of 96 rows (three row tiles: the many-row kernels), then the last row alone
    got = pair.gpu.prefill_last(0, 0, pair.emb[toks])
    want = forward_tokens(pair, 1, toks)[-1]
    assert np.array_equal(bits(got), bits(want))
    # a prefix prefilled, then the rest: the same bits (PrefillTailExact, resident/forward.go:105-109)
    pair.gpu.prefill_last(2, 0, pair.emb[toks[:40]])
    tail = pair.gpu.prefill_last(2, 40, pair.emb[toks[40:]])
    assert np.array_equal(bits(tail), bits(want))
    # against the oracle
    c1, c2 = pair.oracle.new_cache(256), pair.oracle.new_cache(256)
    floor = 0.0
    for p, t in enumerate(toks):
        o = pair.oracle.step(pair.emb[t][None, :], [c1])
        o2 = pair.oracle.step(perturbed(pair.emb[t][None, :], 1e-6, (7, p)), [c2])
        floor = max(floor, float(np.abs(o - o2).max()))
    ok, d = logits_close(got, o[0], floor)
    assert ok, (d, floor)
    # and decode continues from the prefilled slot
    t = ob.argmax(o[0])
    g, _ = pair.gpu.step_batch([0], [97], pair.emb[t][None, :])
    o = pair.oracle.step(pair.emb[t][None, :], [c1])
    o2 = pair.oracle.step(perturbed(pair.emb[t][None, :], 1e-6, (7, 97)), [c2])
    ok, d = logits_close(g[0], o[0], max(floor, float(np.abs(o - o2).max())))
    assert ok, (d, floor)
    pair.close()


VARIANTS = {
    "wide": dense_cfg(n_layers=2, hidden=1024, n_heads=8, n_kv=2, head_dim=128, inter=2560),  # several K ranges a tile, head_dim 128
    "qkv_bias": dict(dense_cfg(n_layers=2, hidden=512, n_heads=8, n_kv=2, head_dim=64, inter=1024, theta=1e6), qkv_bias=1),  # Qwen2: bias in the q|k|v epilogue
    "geglu_post_norms": dict(dense_cfg(n_layers=2, hidden=512, n_heads=8, n_kv=2, head_dim=64, inter=1024, theta=1e4, eps=1e-6, softcap=50.0),
                             window=24, post_norms=1, norm_add_one=1, act_gelu_tanh=1, final_softcap=30.0),  # Gemma 2's block
}


@pytest.mark.parametrize("variant", sorted(VARIANTS))
@pytest.mark.parametrize("n", [70, 150, 300])
def test_many_row_pass_equals_token_by_token(dev, variant, n):
    """A prompt of 65 rows and more goes through the many-row projection kernels (plain, gate|up with SwiGLU or GeGLU, q|k|v with
    bias and RoPE; one or two groups of waves by grid size): the last row's logits and the KV left behind are those of the
    token-by-token path, bit for bit, whatever block variant rides on top."""
    cfg = VARIANTS[variant]
    pair = Pair(cfg, seed=58, dev=dev, slots=2, ctx_cap=n + 8)
    try:
        rng = np.random.default_rng(n)
        toks = list(rng.integers(0, cfg["vocab"], n))
        got = pair.gpu.prefill_last(0, 0, pair.emb[toks])
        want = forward_tokens(pair, 1, toks)[-1]
        assert np.array_equal(bits(got), bits(want))
        for layer in range(cfg["n_layers"]):
            ka, va = pair.gpu.kv_download(0, layer, 0, n)
            kb, vb = pair.gpu.kv_download(1, layer, 0, n)
            assert np.array_equal(bits(ka), bits(kb)) and np.array_equal(bits(va), bits(vb)), layer
        nxt = pair.emb[int(rng.integers(0, cfg["vocab"]))]
        assert np.array_equal(bits(pair.gpu.forward(0, n, nxt)), bits(pair.gpu.forward(1, n, nxt)))
    finally:
        pair.close()


def test_ragged_refusals_write_nothing(dev):
    cfg = dense_cfg()
    pair = Pair(cfg, seed=53, dev=dev, slots=4, ctx_cap=64)
    e = pair.emb[[1, 2, 3]]
    with pytest.raises(capi.RocmError, match="two sequences"):
        pair.gpu.step_ragged([0, 0], [0, 0], [e, e])
    with pytest.raises(capi.RocmError, match="holds 0 rows"):
        pair.gpu.step_ragged([0], [2], [e])
    with pytest.raises(capi.RocmError, match=r"\(-4\)"):  # RD_ERR_KV_FULL: 70 rows do not fit a 64-row slot
        pair.gpu.step_ragged([1], [0], [pair.emb[list(range(70))]])
    with pytest.raises(capi.RocmError, match=r"\(-4\)"):
        pair.gpu.prefill_last(1, 0, pair.emb[list(range(70))])
    # nothing was written: slot 1 still starts at position 0, and its first token equals a fresh slot's
    a = pair.gpu.forward(1, 0, pair.emb[5])
    b = pair.gpu.forward(2, 0, pair.emb[5])
    assert np.array_equal(bits(a), bits(b))
    # a step that names a slot twice without consecutive positions is still refused by the plain batch step
    with pytest.raises(capi.RocmError, match="appears twice"):
        pair.gpu.step_batch([3, 3], [0, 1], pair.emb[[1, 2]])
    pair.close()


def test_forward_no_logits_builds_the_same_kv(dev):
    """ForwardNoLogits skips the head; the K/V it leaves is rd_forward's, so the next token's logits are bit-identical."""
    pair = Pair(dense_cfg(), seed=54, dev=dev, slots=4, ctx_cap=64)
    toks = [5, 77, 300, 12]
    for p, t in enumerate(toks):
        pair.gpu.forward(0, p, pair.emb[t])
        pair.gpu.forward_no_logits(1, p, pair.emb[t])
    a = pair.gpu.forward(0, len(toks), pair.emb[9])
    b = pair.gpu.forward(1, len(toks), pair.emb[9])
    assert np.array_equal(bits(a), bits(b))
    pair.close()


def test_ragged_step_with_draws(dev):
    """A sequence's draw applies to its last row: the argmax, or the host's Gumbel-max token on that row's logits; other rows -1."""
    cfg = dense_cfg(vocab=8192)
    pair = Pair(cfg, seed=55, dev=dev, slots=4, ctx_cap=64)
    rng = np.random.default_rng(4)
    embs = [pair.emb[rng.integers(0, cfg["vocab"], n)] for n in (1, 3, 5, 2)]
    draws = ["greedy", (0.8, 77, 3), None, (1.4, 5 + (9 << 32), 1 << 33)]
    logits, ids = pair.gpu.step_ragged_draw([0, 1, 2, 3], [0, 0, 0, 0], embs, draws, want=capi.WANT_LOGITS)
    last = np.cumsum([len(e) for e in embs]) - 1
    for i, r in enumerate(last):
        if draws[i] is None:
            assert ids[r] == -1
        elif draws[i] == "greedy":
            assert ids[r] == int(np.argmax(logits[r]))
        else:
            assert ids[r] == ob.gumbel_draw(logits[r], *draws[i], guarded=True)
    others = sorted(set(range(len(ids))) - set(int(r) for r in last))
    assert all(ids[r] == -1 for r in others)
    # the logits are those of the plain ragged step on twin state
    pair2 = Pair(cfg, seed=55, dev=dev, slots=4, ctx_cap=64)
    plain, _ = pair2.gpu.step_ragged([0, 1, 2, 3], [0, 0, 0, 0], embs)
    assert np.array_equal(bits(plain), bits(logits))
    pair.close()
    pair2.close()


def test_timed_prompt_pass_leaves_the_prefill_state(dev):
    """rd_bench_prefill (what `bench.py --workload prefill` times) runs rd_prefill_last's passes with the rows looked up on the
    device: the slot it fills continues with the same bits as a slot filled through rd_prefill_last from host rows."""
    from goinfer_amd import synth
    cfg = dense_cfg(n_layers=2, hidden=256, inter=512, vocab=4096)
    pair = Pair(cfg, 47, dev, slots=2, ctx_cap=1152)
    try:
        q, sc = synth.w8a8_normal(78, cfg["vocab"], cfg["hidden"], 0.02)
        rows = q.astype(np.float32) * sc[:, None]
        pair.gpu.upload_embedding(q, sc)
        rng = np.random.default_rng(9)
        toks = rng.integers(0, cfg["vocab"], 1100)  # two full passes of 512 rows, one of 75, the last row alone
        pair.gpu.prefill_last(0, 0, rows[toks])
        ms, classes = pair.gpu.bench_prefill(1, toks, profile=True)
        assert ms > 0 and classes["gemm_qkv"][1] == 4 * cfg["n_layers"]
        nxt = rows[17][None, :]
        a, _ = pair.gpu.step_batch([0], [len(toks)], nxt)
        b, _ = pair.gpu.step_batch([1], [len(toks)], nxt)
        assert np.array_equal(bits(a), bits(b))
    finally:
        pair.close()
