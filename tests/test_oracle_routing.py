"""The oracle's routeExperts / groupLimit and attention sinks / window against the reference's own known answers and against what
the definitions fix.

Known answers: decoder/moe_route_test.go:11-80 (TestRouteExperts): logits [1, 2, 3, 0]; sigmoid scoring with a bias of -5 on
expert 2 picks {1, 0} and weighs them by their UNBIASED sigmoid scores renormalized; the softmax path equals softmax + top-k +
renorm; routed_scaling_factor 2.5 multiplies the weights. groupLimit (decoder/mlp.go:186-228) against a brute-force restatement
in numpy. Sinks and window (decoder/attention.go:57-143, 305-322; kvmgr.WindowNeedStart) against an f64 softmax in numpy.
"""
import math

import numpy as np
import pytest

from goinfer_amd import synth
from oracle import binding as ob


def test_route_experts_known_answers():
    logits = [1, 2, 3, 0]
    idx, wts = ob.route_experts(logits, 2, True, 1.0, bias=[0, 0, -5, 0], sigmoid=True)
    sel = dict(zip(idx.tolist(), wts.tolist()))
    assert 2 not in sel and 0 in sel and 1 in sel  # the highest raw score is biased out of the selection
    s0, s1 = 1 / (1 + math.exp(-1)), 1 / (1 + math.exp(-2))
    assert abs(sel[1] - s1 / (s0 + s1)) <= 1e-5 and abs(sel[0] - s0 / (s0 + s1)) <= 1e-5  # unbiased scores, renormalized
    assert idx.tolist() == [1, 0]  # rank order: the larger selection score first
    # softmax path: softmax + top-k + renorm
    mi, mw = ob.route_experts(logits, 2, True)
    p = np.exp(np.array(logits, np.float64) - 3)
    p /= p.sum()
    assert mi.tolist() == [2, 1]
    assert np.abs(mw - p[[2, 1]] / p[[2, 1]].sum()).max() <= 1e-6
    # routed_scaling_factor multiplies the weights
    _, sw = ob.route_experts(logits, 2, False, 2.5, sigmoid=True)
    _, s1w = ob.route_experts(logits, 2, False, 1.0, sigmoid=True)
    assert np.abs(sw - 2.5 * s1w).max() <= 1e-5


def group_limit_np(sel, n_group, topk_group):
    sel = np.asarray(sel, np.float32)
    gsz = len(sel) // n_group
    gs = np.array([np.float32(np.sort(sel[g * gsz:(g + 1) * gsz])[-1]) + np.float32(np.sort(sel[g * gsz:(g + 1) * gsz])[-2]) if gsz > 1
                   else np.float32(sel[g * gsz]) + np.float32(-np.inf) for g in range(n_group)], np.float32)
    keep = []
    for _ in range(topk_group):  # topK: strict '>', lowest index wins, -inf never
        best, bi = -np.inf, -1
        for g in range(n_group):
            if g not in keep and gs[g] > best:
                best, bi = gs[g], g
        if bi < 0:
            break
        keep.append(bi)
    out = np.full(len(sel), -np.inf, np.float32)
    for g in keep:
        out[g * gsz:(g + 1) * gsz] = sel[g * gsz:(g + 1) * gsz]
    return out


@pytest.mark.parametrize("nE,n_group,topk_group", [(8, 4, 2), (64, 8, 3), (128, 8, 4), (30, 4, 2), (16, 16, 5)])
def test_group_limit_matches_brute_force(nE, n_group, topk_group):
    rng = np.random.default_rng(nE + n_group)
    for trial in range(20):
        sel = rng.standard_normal(nE).astype(np.float32)
        if trial % 4 == 0:
            sel = np.round(sel * 2) / 2  # ties between groups and inside them
        got = ob.group_limit(sel, n_group, topk_group)
        want = group_limit_np(sel, n_group, topk_group)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        # and through routeExperts: every pick lies in a kept group, the trailing experts of an uneven split never win
        idx, _ = ob.route_experts(sel, min(6, nE), False, bias=np.zeros(nE, np.float32), sigmoid=True, n_group=n_group, topk_group=topk_group)
        sig = (1.0 / (1.0 + np.exp(-sel.astype(np.float64)))).astype(np.float32)
        lim = group_limit_np(sig, n_group, topk_group)
        assert all(np.isfinite(lim[i]) for i in idx)


def attend_np(q, keys, vals, n, nH, nKV, hd, scale, softcap, start, sinks):
    out = np.zeros((nH, hd))
    G = nH // nKV
    for h in range(nH):
        kv = h // G
        K = keys[:n, kv * hd:(kv + 1) * hd].astype(np.float64)
        V = vals[:n, kv * hd:(kv + 1) * hd].astype(np.float64)
        s = K @ q[h * hd:(h + 1) * hd].astype(np.float64) * scale
        if softcap:
            s = softcap * np.tanh(s / softcap)
        s = s[start:]
        m = s.max()
        if sinks is not None:
            m = max(m, float(sinks[h]))
        e = np.exp(s - m)
        den = e.sum() + (math.exp(float(sinks[h]) - m) if sinks is not None else 0.0)
        out[h] = (e / den) @ V[start:]
    return out.reshape(-1)


@pytest.mark.parametrize("softcap", [0.0, 5.0])
def test_attend_sinks_and_window(softcap):
    nH, nKV, hd, n = 8, 2, 32, 50
    q = synth.normal(1, nH * hd)
    keys = synth.normal(2, n * nKV * hd).reshape(n, nKV * hd)
    vals = synth.normal(3, n * nKV * hd).reshape(n, nKV * hd)
    sinks = synth.normal(4, nH, 3.0)
    scale = hd ** -0.5
    for start, sk in ((0, None), (0, sinks), (37, None), (46, sinks), (49, sinks)):
        got = ob.attend(q, keys, vals, n, nH, nKV, hd, scale, softcap, start=start, sinks=sk)
        want = attend_np(q, keys, vals, n, nH, nKV, hd, scale, softcap, start, sk)
        assert np.abs(got - want).max() <= 2e-6 * max(1.0, np.abs(want).max())
    # a sink takes probability mass away: the output shrinks toward zero and never grows
    a = ob.attend(q, keys, vals, n, nH, nKV, hd, scale, softcap)
    b = ob.attend(q, keys, vals, n, nH, nKV, hd, scale, softcap, sinks=np.full(nH, 50.0, np.float32))
    assert np.abs(b).max() < 1e-6 * np.abs(a).max() + 1e-12
