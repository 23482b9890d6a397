"""The step's launches replayed from a captured HIP graph give the bits the eager launches give.

Every replay is checked against a twin model that never uses a graph, with eager work of the program's own (cache reads, steps of
another shape, resets) and synchronizations between the replays, over steps whose work list keeps its size (replayed) and steps
where it changes (launched eagerly, then captured anew)."""
import numpy as np
import pytest

from goinfer_amd import capi, synth
from tests.models import Pair, dense_cfg, moe_cfg

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = capi.Device(0)
    yield d
    d.close()


def twins(cfg, seed, dev, **kw):
    a, b = Pair(cfg, seed=seed, dev=dev, **kw), Pair(cfg, seed=seed, dev=dev, **kw)
    b.gpu.set_graph(False)
    return a, b


def same_bits(x, y):
    return np.array_equal(np.asarray(x).view(np.uint32), np.asarray(y).view(np.uint32))


@pytest.mark.parametrize("name,cfg,B,steps", [("dense", dense_cfg(n_layers=3), 5, 150), ("dense two M-tiles", dense_cfg(n_layers=2), 40, 330),
                                              ("moe", moe_cfg(), 6, 150),
                                              ("windowed", dict(dense_cfg(n_layers=4), window=24, attn_sinks=1), 4, 150)])
def test_graph_replays_equal_eager_steps(dev, name, cfg, B, steps):
    a, b = twins(cfg, 5, dev, slots=max(B, 8), ctx_cap=512)
    try:
        rng = np.random.default_rng(9)
        slots = list(range(B))
        for p in range(steps):  # the positions cross block boundaries every 64: the work list grows there
            toks = rng.integers(0, cfg["vocab"], B)
            want = capi.WANT_LOGITS | capi.WANT_ARGMAX
            la, ia = a.gpu.step_batch(slots, [p] * B, a.emb[toks], want)
            lb, ib = b.gpu.step_batch(slots, [p] * B, b.emb[toks], want)
            assert same_bits(la, lb) and np.array_equal(ia, ib), (name, p)
            if p % 7 == 3:  # eager work of the program's own between two replays
                ka, va = a.gpu.kv_download(0, 0, 0, p + 1)
                kb, vb = b.gpu.kv_download(0, 0, 0, p + 1)
                assert same_bits(ka, kb) and same_bits(va, vb)
            if p % 31 == 30 and B < 8:  # a one-row step on a spare slot in between: another key, launched eagerly
                for m in (a, b):
                    m.spare = m.gpu.step_batch([7], [p // 31], m.emb[toks[:1]])[0]
                assert same_bits(a.spare, b.spare)
        caps, reps = a.gpu.graph_stats()
        assert caps >= 1 and reps >= 100, (caps, reps)  # most steps ran from a graph
        if B == 40:  # 80 (row, kv head) pairs x 4 pieces outgrow the 256 items the launch was padded to: a new graph
            assert caps >= 2, caps
        assert b.gpu.graph_stats() == (0, 0)
    finally:
        a.close()
        b.close()


def test_graph_survives_steps_of_other_shapes_between_replays(dev):
    """Full-batch steps replay a graph; between them steps of another batch size and a ragged step run eagerly on the same
    buffers; the next full-batch step must not replay stale launches (its work list has grown)."""
    cfg = dense_cfg(n_layers=2)
    a, b = twins(cfg, 6, dev, slots=8, ctx_cap=256)
    try:
        rng = np.random.default_rng(10)
        pos = [0, 0, 0, 0]
        for it in range(40):
            for m in (a, b):
                m.out = []
            toks = rng.integers(0, 512, 4)
            extra = rng.integers(0, 512, 3)
            for m in (a, b):
                m.out.append(m.gpu.step_batch([0, 1, 2, 3], pos, m.emb[toks])[0])
            pos = [p + 1 for p in pos]
            if it % 5 == 4:  # slot 4 takes three positions in one ragged step, then one plain step of batch 1
                base = 3 * (it // 5) + (it // 5)
                for m in (a, b):
                    m.out.append(m.gpu.step_ragged([4], [base], [m.emb[extra]])[0])
                    m.out.append(m.gpu.step_batch([4], [base + 3], m.emb[extra[:1]])[0])
            for x, y in zip(a.out, b.out):
                assert same_bits(x, y), it
        caps, reps = a.gpu.graph_stats()
        assert reps >= 20, (caps, reps)
    finally:
        a.close()
        b.close()


def test_graph_in_a_device_chain(dev):
    """The device-chained greedy decode queues steps ahead of the host; with the graph on it gives the ids it gives without."""
    cfg = dense_cfg(n_layers=2, vocab=512)
    a, b = twins(cfg, 7, dev, slots=2, ctx_cap=512)
    try:
        q, sc = synth.w8a8_normal(77, cfg["vocab"], cfg["hidden"], 0.02)
        ids = []
        for m in (a, b):
            m.gpu.upload_embedding(q, sc)
            m.gpu.greedy_chain_start(0, 17, 0)
            ids.append([m.gpu.greedy_chain_next() for _ in range(200)])
            m.gpu.chain_stop()
        assert ids[0] == ids[1]
        caps, reps = a.gpu.graph_stats()
        assert reps >= 150, (caps, reps)
    finally:
        a.close()
        b.close()


def test_draw_steps_and_switching_the_graph_off(dev):
    """Steps with per-row draws have a graph of their own (the argmax kernel reads the draw records); switching the graph off in
    the middle of a run changes nothing."""
    cfg = dense_cfg(n_layers=2)
    a, b = twins(cfg, 8, dev, slots=4, ctx_cap=256)
    try:
        rng = np.random.default_rng(11)
        for p in range(30):
            toks = rng.integers(0, 512, 3)
            draws = ["greedy", (0.8, 1234, p), None]
            if p == 20:
                a.gpu.set_graph(False)
            for m in (a, b):
                m.o1 = m.gpu.step_batch_draw([0, 1, 2], [p] * 3, m.emb[toks], draws, capi.WANT_LOGITS)
            assert same_bits(a.o1[0], b.o1[0]) and np.array_equal(a.o1[1], b.o1[1]), p
        caps, reps = a.gpu.graph_stats()
        assert caps >= 1 and 10 <= reps <= 19, (caps, reps)
    finally:
        a.close()
        b.close()


def test_a_changed_kernel_knob_is_never_served_by_an_older_graph(dev):
    """The environment knobs that pick kernels (waves per GEMM tile, splits, attention kernel, fused epilogues) are part of what a
    captured graph was recorded for: the step after a change is launched anew, not replayed, and equals the twin that never
    uses a graph under the same knob; replays are counted only when the graph launch went through."""
    import os
    cfg = dense_cfg(n_layers=2, hidden=512, n_heads=4, n_kv=2, head_dim=128, inter=1024)
    a, b = twins(cfg, 7, dev, slots=4, ctx_cap=64)
    try:
        rng = np.random.default_rng(3)
        pos = 0

        def step():
            nonlocal pos
            toks = rng.integers(0, cfg["vocab"], 4)
            la = a.gpu.step_batch([0, 1, 2, 3], [pos] * 4, a.emb[toks])[0]
            lb = b.gpu.step_batch([0, 1, 2, 3], [pos] * 4, b.emb[toks])[0]
            pos += 1
            assert same_bits(la, lb), pos

        for _ in range(4):
            step()
        caps0, reps0 = a.gpu.graph_stats()
        assert caps0 == 1 and reps0 == 2  # eager, captured (which runs the step), replayed, replayed
        for knob, val in (("ROCMDECODE_GEMM8_KW", "2"), ("ROCMDECODE_GEMM8_SPLITS", "2"), ("ROCMDECODE_NO_DEEP_ATTN", "1"), ("ROCMDECODE_NO_ROWS_GEMM", "1")):
            os.environ[knob] = val
            try:
                before = a.gpu.graph_stats()
                step()  # a new key: launched eagerly
                assert a.gpu.graph_stats() == before, knob
                step()  # the second step under the knob is captured
                step()
                assert a.gpu.graph_stats() == (before[0] + 1, before[1] + 1), knob
            finally:
                del os.environ[knob]
            step()  # and back: a new key again
    finally:
        a.close()
        b.close()


@pytest.mark.parametrize("name,cfg", [("hidden 256", dense_cfg(n_layers=3)), ("hidden 1024, biases", dict(dense_cfg(n_layers=2, hidden=1024, n_heads=8, n_kv=2, head_dim=128, inter=1536), qkv_bias=1)),
                                      ("hidden 4096", dense_cfg(n_layers=2, hidden=4096, n_heads=8, n_kv=2, head_dim=128, inter=2048))])
def test_one_row_steps_with_the_norm_folded_into_the_projections_equal_the_separate_kernels(dev, name, cfg):
    """A step of one row forms the row's norm and quantization inside its q|k|v and gate|up projections (one launch less each); with
    ROCMDECODE_NO_FUSED_NORM the norm kernel is launched on its own as in a batch. Both, eager and replayed from a graph, give the
    same logits bit for bit, position after position (the residual row alternates between two buffers in the folded form), and the
    row equals the same sequence's row in a batch of two."""
    import os
    a, b = twins(cfg, 11, dev, slots=4, ctx_cap=256)
    c, d = Pair(cfg, seed=11, dev=dev, slots=4, ctx_cap=256), Pair(cfg, seed=11, dev=dev, slots=4, ctx_cap=256)
    try:
        rng = np.random.default_rng(5)
        for p in range(70):  # crosses a 64-position block boundary
            tok = rng.integers(0, cfg["vocab"], 2)
            la = a.gpu.step_batch([0], [p], a.emb[tok[:1]])[0]  # folded, replayed from a graph after the second step
            lb = b.gpu.step_batch([0], [p], b.emb[tok[:1]])[0]  # folded, eager
            os.environ["ROCMDECODE_NO_FUSED_NORM"] = "1"
            try:
                lc = c.gpu.step_batch([0], [p], c.emb[tok[:1]])[0]  # the norm kernel on its own
            finally:
                del os.environ["ROCMDECODE_NO_FUSED_NORM"]
            ld = d.gpu.step_batch([0, 1], [p, p], d.emb[tok])[0]  # the same sequence as row 0 of a batch of two
            assert same_bits(la, lb), (name, p)
            assert same_bits(la, lc), (name, p)
            assert same_bits(la[0], ld[0]), (name, p)
        assert a.gpu.graph_stats()[1] > 40
    finally:
        for m in (a, b, c, d):
            m.close()
