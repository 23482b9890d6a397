"""The oracle's restatement of the K best logits of a row (internal/runtime/sampling/sampler.go:726-782 topKByLogit, in the order
resident.TopKRow promises) and of the top-p denominator, against what their definitions fix: the first K of the row under
(logit descending, id ascending) is unique, so an independent full sort must give the same ids in the same order. The row shapes
are those of the reference's own device test (backend/cuda/topk_test.go:24-125): normal logits, rows of a few distinct values so
that the cut runs through ties, signed zeros, K from 1 up to the whole row."""
import numpy as np
import pytest

from oracle import binding as ob


def sorted_reference(x, k):
    """Full sort by (value descending, id ascending) with -0 equal to +0."""
    canon = np.where(x == 0, np.float32(0), x).astype(np.float32)
    order = np.lexsort((np.arange(x.size), -canon.astype(np.float64)))
    return order[:k].astype(np.int32)


def rows(n, seed):
    rng = np.random.default_rng(seed)
    normal = rng.standard_normal(n).astype(np.float32) * 3
    tied = rng.integers(0, 9, n).astype(np.float32)
    zeros = np.where(rng.random(n) < 0.5, np.float32(0.0), np.float32(-0.0)).astype(np.float32)
    zeros[rng.integers(0, n, max(1, n // 50))] = 1.5
    ramp = np.arange(n, dtype=np.float32)[::-1].copy()
    const = np.full(n, -2.25, np.float32)
    return {"normal": normal, "tied": tied, "signed zeros": zeros, "descending": ramp, "constant": const}


@pytest.mark.parametrize("n", [1, 7, 64, 1000, 5003])
def test_topk_by_logit_is_the_sorted_prefix(n):
    for name, x in rows(n, 100 + n).items():
        for k in sorted({1, 2, min(n, 37), min(n, 256), n}):
            ids, vals = ob.topk_by_logit(x, k)
            want = sorted_reference(x, min(k, n))
            assert np.array_equal(ids, want), (name, n, k)
            assert np.array_equal(vals.view(np.uint32), x[want].view(np.uint32)), (name, n, k)  # the entries' own bits, -0 included
    ids, _ = ob.topk_by_logit(np.array([1, 3, 3, 2], np.float32), 10)  # k beyond the row: the whole row, ordered
    assert ids.tolist() == [1, 2, 3, 0]


@pytest.mark.parametrize("T", [0.3, 1.0, 2.5])
def test_softmax_z(T):
    x = (np.random.default_rng(5).standard_normal(4096) * 4).astype(np.float32)
    want = np.exp((x.astype(np.float64) - float(x.max())) / T).sum()
    assert abs(ob.softmax_z(x, T) - want) <= 1e-12 * want
    assert ob.softmax_z(np.array([2.0], np.float32), T) == 1.0
