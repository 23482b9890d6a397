"""Device-side draws against the oracle's restatement of goinfer's host sampler (internal/runtime/sampling/sampler_gumbel.go).

The draw is a pure function of (logits, temperature, seed, draw): Philox words are integer-exact and the noise transform is
evaluated in f64 on both sides, so the bar is identity of the drawn token with the oracle's on the same logits. (The
reference's own CUDA kernel computes the transform in f32 and tolerates disagreement when the two best keys are a few ulps
apart, backend/cuda/gumbel.cu:5-8; nothing is tolerated here.)"""
import numpy as np
import pytest

from goinfer_amd import capi
from oracle import binding as ob
from tests.models import Pair, dense_cfg

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = capi.Device(0)
    yield d
    d.close()


@pytest.mark.parametrize("V", [7, 63, 4099, 32768, 151936])
def test_sample_rows_equals_host_draw(dev, V):
    """The vocabulary sizes and temperatures of the reference's TestGumbelDraw_parallelEqualsSequential."""
    rng = np.random.default_rng(V)
    rows = 24
    logits = (rng.standard_normal((rows, V)) * 3).astype(np.float32)
    draws = []
    for r in range(rows):
        T = (0.3, 1.0, 2.5)[r % 3]
        draws.append((T, 99 + (r << 33), r * 7 + (1 << 40) * (r % 2)))  # seeds and draws that use their high words
    got = dev.sample_rows(logits, draws)
    want = [ob.gumbel_draw(logits[r], *draws[r], guarded=True) for r in range(rows)]
    assert list(got) == want


def test_sample_rows_edges(dev):
    V = 64
    l = np.full((5, V), -np.inf, np.float32)
    l[0, 17], l[0, 40] = 0.0, 0.5          # -Inf is never drawn
    l[2] = np.arange(V, dtype=np.float32)  # tiny temperature: the argmax; temperature <= 0: as 1
    l[3] = np.arange(V, dtype=np.float32) * 0.01
    l[4] = 1.5                             # flat row, greedy: first index
    draws = [(1.0, 3, 0), (1.0, 3, 1), (1e-40, 1, 0), (0.0, 21, 3), "greedy"]
    got = dev.sample_rows(l, draws)
    assert got[0] in (17, 40)
    assert got[1] == 0  # a fully masked row falls back to the argmax, index 0
    assert got[2] == V - 1
    assert got[3] == ob.gumbel_draw(l[3], 1.0, 21, 3)
    assert got[4] == 0
    many = dev.sample_rows(np.repeat(l[:1], 32, axis=0), [(1.0, 5, d) for d in range(32)])
    assert set(many) <= {17, 40} and len(set(many)) == 2


def test_step_batch_draw(dev):
    """The step's own draws: greedy rows return the argmax of the logits the row returns, temperature rows the host's draw
    on those logits, rows without a draw -1; logits are bit-identical to a step without draws."""
    cfg = dense_cfg(n_layers=2, hidden=256, inter=512, vocab=12288)  # three 4096-column chunks
    pair = Pair(cfg, 41, dev, slots=8, ctx_cap=64)
    try:
        rng = np.random.default_rng(2)
        B = 6
        for step in range(4):
            toks = rng.integers(0, cfg["vocab"], B)
            emb = pair.emb[toks]
            draws = [None, "greedy", (0.7, 11, step), (1.3, 12 + (5 << 32), step + (1 << 35)), (1e-40, 1, step), (0.0, 9, step)]
            logits, ids = pair.gpu.step_batch_draw(list(range(B)), [step] * B, emb, draws, want=capi.WANT_LOGITS)
            assert ids[0] == -1
            assert ids[1] == int(np.argmax(logits[1]))
            for b in (2, 3, 4, 5):
                assert ids[b] == ob.gumbel_draw(logits[b], *draws[b], guarded=True), (step, b)
            # the same rows on twin slots through the plain step: identical logits
            plain, _ = pair.gpu.step_batch([B], [step], emb[:1])
            assert np.array_equal(plain[0].view(np.uint32), logits[0].view(np.uint32))
            _, ids_only = pair.gpu.step_batch_draw([7], [step], emb[2:3], [draws[2]])
            assert ids_only[0] == ids[2]  # without the logits readback the draw is the same
        with pytest.raises(capi.RocmError):
            pair.gpu.step_batch_draw([0], [4], pair.emb[:1], [(float("nan"), 1, 1)])
    finally:
        pair.close()


def int8_table(seed, V, H):
    """An int8 embedding table with per-row scales, and the f32 rows the host's lookup would send for it."""
    from goinfer_amd import synth
    q, sc = synth.w8a8_normal(seed, V, H, 0.02)
    return q, sc, q.astype(np.float32) * sc[:, None]


def test_greedy_and_sample_chain_equal_host_driven_steps(dev):
    """The chained tokens are those of the host-driven loop: step, read logits, pick, look the row up, step again."""
    cfg = dense_cfg(n_layers=2, hidden=256, inter=512, vocab=4096)
    pair = Pair(cfg, 43, dev, slots=4, ctx_cap=48)
    try:
        q, sc, rows = int8_table(77, cfg["vocab"], cfg["hidden"])
        pair.gpu.upload_embedding(q, sc)
        prompt = [5, 99, 1234, 7]
        n = 20
        # host-driven reference on slot 0 (greedy) and slot 1 (temperature 0.8, seed 5, draws 100...)
        for p, t in enumerate(prompt[:-1]):
            for s in (0, 1, 2, 3):
                pair.gpu.step_batch([s], [p], rows[t][None, :])
        host_g, host_s = [], []
        tg = ts = prompt[-1]
        for i in range(n):
            lg, _ = pair.gpu.step_batch([0], [len(prompt) - 1 + i], rows[tg][None, :])
            tg = int(np.argmax(lg[0]))
            host_g.append(tg)
            ls, _ = pair.gpu.step_batch([1], [len(prompt) - 1 + i], rows[ts][None, :])
            ts = ob.gumbel_draw(ls[0], 0.8, 5, 100 + i, guarded=True)
            host_s.append(ts)
        # chained on slots 2 and 3
        pair.gpu.greedy_chain_start(2, prompt[-1], len(prompt) - 1)
        with pytest.raises(capi.RocmError):
            pair.gpu.step_batch([0], [0], rows[:1])  # no other step while a chain is open
        got_g = [pair.gpu.greedy_chain_next() for _ in range(n)]
        pair.gpu.chain_stop()
        assert got_g == host_g
        pair.gpu.sample_chain_start(3, prompt[-1], len(prompt) - 1, 0.8, 5, 100)
        got_s = []
        for i in range(n):
            if i == 3:
                with pytest.raises(capi.RocmError):
                    pair.gpu.sample_chain_next(5, 999)  # not the draw this forward was made with
            got_s.append(pair.gpu.sample_chain_next(5, 100 + i))
        pair.gpu.chain_stop()
        assert got_s == host_s
        assert len(set(got_s)) > 3
        # after a chain the slot continues from the host: the token the chain returned last, at the next position
        lg, _ = pair.gpu.step_batch([2], [len(prompt) - 1 + n], rows[got_g[-1]][None, :])
        l0, _ = pair.gpu.step_batch([0], [len(prompt) - 1 + n], rows[host_g[-1]][None, :])
        assert np.array_equal(lg.view(np.uint32), l0.view(np.uint32))
    finally:
        pair.close()


def test_chain_runs_into_the_context_cap(dev):
    cfg = dense_cfg(n_layers=1, hidden=256, inter=512, vocab=512)
    pair = Pair(cfg, 44, dev, slots=2, ctx_cap=8)
    try:
        q, sc, rows = int8_table(78, cfg["vocab"], cfg["hidden"])
        with pytest.raises(capi.RocmError):
            pair.gpu.greedy_chain_start(0, 1, 0)  # no embedding table yet
        pair.gpu.upload_embedding(q, sc)
        pair.gpu.greedy_chain_start(0, 1, 0)
        toks = [pair.gpu.greedy_chain_next() for _ in range(8)]  # positions 0..7 fit
        assert all(0 <= t < 512 for t in toks)
        with pytest.raises(capi.RocmError) as ei:
            pair.gpu.greedy_chain_next()  # position 8 is the cap: the look-ahead could not be queued
        assert "(-4)" in str(ei.value)
        pair.gpu.chain_stop()
        pair.gpu.kv_reset(0)
        pair.gpu.step_batch([0], [0], rows[:1])
    finally:
        pair.close()


def test_tied_keys_at_tiny_temperatures_keep_the_host_order(dev):
    """Two equal largest logits at a temperature so small that the noise vanishes in the f32 key: the keys tie and the lowest
    index wins, as on the host. The product logit * 1/T must be rounded before the noise is added (sampler_gumbel.go:41-66): a
    fused multiply-add lets the noise's sign decide the rounding of a product that falls halfway between two f32 values, and
    the tie breaks the other way."""
    seed, draw = 4648040972980819852, 2410598768476298352
    V = 211
    row = np.full(V, -3.0, np.float32)
    row[107] = row[115] = 6.0
    for T in (1e-30, 1e-25, 1e-20, 1e-10, 1e-6, 1e-3, 1.0):
        got = dev.sample_rows(row[None, :], [(T, seed, draw)])
        assert int(got[0]) == ob.gumbel_draw(row, T, seed, draw, guarded=True), T
    rng = np.random.default_rng(5)
    rows = np.round(rng.standard_normal((64, 300)) * 2).astype(np.float32)  # heavily tied rows
    draws = [((1e-30, 1e-10, 1e-8, 3e-7)[r % 4], int(rng.integers(0, 1 << 62)), r) for r in range(64)]
    got = dev.sample_rows(rows, draws)
    assert list(got) == [ob.gumbel_draw(rows[r], *draws[r], guarded=True) for r in range(64)]
