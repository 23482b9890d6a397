"""The device-side top-K of a logits row (rd_topk_rows, rd_step_batch_topk; goinfer's resident.TopKRow / ForwardTopK,
decoder/resident/forward.go:86-96, backend/cuda/topk.go:30-110) against the oracle's topKByLogit.

Bars, the reference's own (backend/cuda/topk_test.go:24-125): ids and logit bits identical to the reference order (logit
descending, id ascending; -0 and +0 tie) on normal, heavily tied and flat rows, for vocabularies from below a block to 152k and
K from 1 to 1024; Z within 1e-6 relative of the f64 sum. Rows of 32768 entries and more go over the chip in three launches
(histogram, candidates, sort); of the shapes here only the normal rows fit the candidate list, the tied and flat ones take the
exact one-block selection inside the last launch: both routes are held to the same order."""
import numpy as np
import pytest

from goinfer_amd import capi
from oracle import binding as ob
from tests.models import Pair, dense_cfg
from tests.test_oracle_topk import rows

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = capi.Device(0)
    yield d
    d.close()


@pytest.mark.parametrize("V", [5, 64, 1000, 8192, 32000, 32768, 100003, 151936])
def test_topk_rows_match_the_reference_order(dev, V):
    shapes = rows(V, 7 + V)
    names = list(shapes)
    x = np.stack([shapes[n] for n in names])
    for k in sorted({1, min(V, 40), min(V, 256), min(V, 1024)}):
        for T in (0.7,):
            ids, vals, z = dev.topk_rows(x, k, T)
            for r, name in enumerate(names):
                wi, wv = ob.topk_by_logit(x[r], k)
                assert np.array_equal(ids[r], wi), (name, V, k)
                assert np.array_equal(vals[r].view(np.uint32), wv.view(np.uint32)), (name, V, k)
                zw = ob.softmax_z(x[r], T)
                assert abs(z[r] - zw) <= 1e-6 * zw, (name, V, k, z[r], zw)
    again = dev.topk_rows(x, min(V, 256), 0.7)
    first = dev.topk_rows(x, min(V, 256), 0.7)
    assert np.array_equal(again[0], first[0]) and np.array_equal(again[2].view(np.uint64), first[2].view(np.uint64))


@pytest.mark.parametrize("V", [3000, 70000])
def test_topk_rows_with_masked_entries(dev, V):
    """Rows a logit processor has masked: most entries -Inf (never in the top while finite ones remain, tied among themselves by
    id when K reaches into them) and Z counts them as zero."""
    rng = np.random.default_rng(V)
    x = np.full((2, V), -np.inf, np.float32)
    keep = rng.choice(V, 300, replace=False)
    x[0, keep] = rng.standard_normal(300).astype(np.float32) * 2
    x[1, keep[:5]] = np.float32(1.25)  # five equal finite entries, the rest masked
    for k in (1, 5, 200, 512):
        ids, vals, z = dev.topk_rows(x, k, 0.9)
        for r in range(2):
            wi, wv = ob.topk_by_logit(x[r], k)
            assert np.array_equal(ids[r], wi), (V, k, r)
            assert np.array_equal(vals[r].view(np.uint32), wv.view(np.uint32))
            zw = ob.softmax_z(x[r], 0.9)
            assert abs(z[r] - zw) <= 1e-6 * zw


def test_topk_rows_arguments(dev):
    x = np.zeros((1, 100), np.float32)
    with pytest.raises(capi.RocmError):
        dev.topk_rows(x, 0)
    with pytest.raises(capi.RocmError):
        dev.topk_rows(x, 1025)
    ids, vals, z = dev.topk_rows(x, 1024, want_z=False)  # k beyond the row: the whole row, ids ascending on the all-equal row
    assert z is None and ids.shape == (1, 100) and ids[0].tolist() == list(range(100))


def test_step_batch_topk_is_the_top_of_the_steps_logits(dev):
    """The step's own logits row, reduced: the entries equal the oracle's top-K of the logits rd_step_batch returns for the same
    rows, Z is that row's denominator at the row's temperature, and rd_last_logits hands the whole row back (TopKRow.Full)."""
    cfg = dense_cfg(n_layers=2, vocab=4096)
    pair = Pair(cfg, seed=91, dev=dev, slots=8, ctx_cap=32)
    try:
        rng = np.random.default_rng(3)
        B = 3
        toks = rng.integers(0, cfg["vocab"], B)
        full, _ = pair.gpu.step_batch([0, 1, 2], [0, 0, 0], pair.emb[toks])
        temps = [0.5, 1.0, 1.7]
        ids, vals, z = pair.gpu.step_batch_topk([4, 5, 6], [0, 0, 0], pair.emb[toks], 50, temps)
        for b in range(B):
            wi, wv = ob.topk_by_logit(full[b], 50)
            assert np.array_equal(ids[b], wi) and np.array_equal(vals[b].view(np.uint32), wv.view(np.uint32))
            zw = ob.softmax_z(full[b], temps[b])
            assert abs(z[b] - zw) <= 1e-6 * zw
            assert np.array_equal(pair.gpu.last_logits(b).view(np.uint32), full[b].view(np.uint32))
        ids1, vals1, z1 = pair.gpu.step_batch_topk([7], [0], pair.emb[toks[:1]], 8)  # ForwardTopK without Z
        assert z1 is None and np.array_equal(ids1[0], ids[0][:8])
        with pytest.raises(capi.RocmError):
            pair.gpu.last_logits(1)  # the last step had one row
    finally:
        pair.close()
