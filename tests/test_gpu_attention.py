"""Ragged flash-decode attention on the GPU against the oracle's f64-accumulated attention (goinfer forwardn.go:295-500),
through rd_attn_ragged. Bar: the reference's own flash-decode bar, rel-err <= 1e-4 against the f64 oracle
(backend/cuda/flash_decode_test.go:56-150), plus run-to-run bit determinism."""
import numpy as np
import pytest

from goinfer_amd import capi, synth
from oracle import binding as ob

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = capi.Device(0)
    yield d
    d.close()


def f16_round_trip(x):
    """What the cache stores: binary16 with round-half-up, widened back (the oracle's own conversion)."""
    L = ob.lib()
    flat = x.ravel()
    out = np.empty_like(flat)
    for i, v in enumerate(flat):
        out[i] = L.or_f16_to_f32(L.or_f32_to_f16(float(v)))
    return out.reshape(x.shape)


def oracle_attn(lens, k, v, q, nH, nKV, hd, scale, softcap):
    out = np.empty((len(lens), nH * hd), np.float32)
    off = 0
    for i, n in enumerate(lens):
        out[i] = ob.attend(q[i], k[off:off + n], v[off:off + n], n, nH, nKV, hd, scale, softcap)
        off += n
    return out


@pytest.mark.parametrize("hd", [64, 128])
@pytest.mark.parametrize("nH,nKV", [(4, 1), (8, 8), (14, 2)])
@pytest.mark.parametrize("softcap", [0.0, 50.0])
def test_ragged_attention_small(dev, hd, nH, nKV, softcap):
    lens = [1, 7, 8, 9, 63, 64, 65, 300]
    tot, kvd = sum(lens), nKV * hd
    k = synth.normal(1, tot * kvd).reshape(tot, kvd)
    v = synth.normal(2, tot * kvd).reshape(tot, kvd)
    q = synth.normal(3, len(lens) * nH * hd).reshape(len(lens), nH * hd)
    scale = float(1.0 / np.sqrt(hd))
    got = dev.attn_ragged(lens, k, v, q, nH, nKV, hd, scale, softcap)
    want = oracle_attn(lens, f16_round_trip(k), f16_round_trip(v), q, nH, nKV, hd, scale, softcap)
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err <= 1e-4, err
    again = dev.attn_ragged(lens, k, v, q, nH, nKV, hd, scale, softcap)
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))


def test_ragged_attention_long_split(dev):
    """Lengths past the split threshold (several work items per (sequence, kv head)), 32q/8kv hd128 as the benchmark shape."""
    lens = [1000, 4097, 128, 2050]
    nH, nKV, hd = 32, 8, 128
    tot, kvd = sum(lens), nKV * hd
    rng = np.random.default_rng(5)
    k = rng.standard_normal((tot, kvd), dtype=np.float32).astype(np.float16).astype(np.float32)
    v = rng.standard_normal((tot, kvd), dtype=np.float32).astype(np.float16).astype(np.float32)
    q = rng.standard_normal((len(lens), nH * hd), dtype=np.float32)
    scale = float(1.0 / np.sqrt(hd))
    for softcap in (0.0, 50.0):
        got = dev.attn_ragged(lens, k, v, q, nH, nKV, hd, scale, softcap)
        want = oracle_attn(lens, k, v, q, nH, nKV, hd, scale, softcap)
        err = np.abs(got - want).max() / np.abs(want).max()
        assert err <= 1e-4, (softcap, err)


def test_softcap_changes_result_and_matches_closed_form(dev):
    """Large scores so the cap bites: out = softmax(cap*tanh(s/cap)) . V against numpy float64."""
    n, nH, nKV, hd = 130, 4, 2, 64
    rng = np.random.default_rng(9)
    k = (4 * rng.standard_normal((n, nKV * hd))).astype(np.float16).astype(np.float32)
    v = rng.standard_normal((n, nKV * hd)).astype(np.float16).astype(np.float32)
    q = (4 * rng.standard_normal((1, nH * hd))).astype(np.float32)
    cap, scale = 5.0, 0.125
    got = dev.attn_ragged([n], k, v, q, nH, nKV, hd, scale, cap)[0]
    plain = dev.attn_ragged([n], k, v, q, nH, nKV, hd, scale, 0.0)[0]
    assert np.abs(got - plain).max() > 1e-2
    for h in range(nH):
        kv = h // (nH // nKV)
        s = k[:, kv * hd:(kv + 1) * hd].astype(np.float64) @ q[0, h * hd:(h + 1) * hd].astype(np.float64) * scale
        s = cap * np.tanh(s / cap)
        p = np.exp(s - s.max())
        p /= p.sum()
        want = p @ v[:, kv * hd:(kv + 1) * hd].astype(np.float64)
        assert np.abs(got[h * hd:(h + 1) * hd] - want).max() <= 2e-4 * max(1.0, np.abs(want).max())


def i8_round_trip(x, nKV, hd):
    """What the int8 cache holds of K or V rows [n][nKV*hd]: per head the codes times their scale (the oracle's own functions,
    both pinned by the reference's fingerprints)."""
    heads = x.reshape(-1, hd)
    q, sc = ob.quantize_rows_int8(heads)
    return ob.dequantize_rows_int8(q, sc).reshape(x.shape)


@pytest.mark.parametrize("hd", [64, 128])
@pytest.mark.parametrize("nH,nKV", [(4, 1), (8, 8), (14, 2)])
@pytest.mark.parametrize("softcap", [0.0, 50.0])
def test_ragged_attention_i8_small(dev, hd, nH, nKV, softcap):
    """The int8 cache: the same bar against the oracle's attention over the dequantized rows."""
    lens = [1, 7, 8, 9, 63, 64, 65, 300]
    tot, kvd = sum(lens), nKV * hd
    k = synth.normal(1, tot * kvd).reshape(tot, kvd)
    v = synth.normal(2, tot * kvd).reshape(tot, kvd)
    k[5] = 0.0  # an all-zero row: scale 1, codes 0
    q = synth.normal(3, len(lens) * nH * hd).reshape(len(lens), nH * hd)
    scale = float(1.0 / np.sqrt(hd))
    got = dev.attn_ragged(lens, k, v, q, nH, nKV, hd, scale, softcap, kv="i8")
    want = oracle_attn(lens, i8_round_trip(k, nKV, hd), i8_round_trip(v, nKV, hd), q, nH, nKV, hd, scale, softcap)
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err <= 1e-4, err
    again = dev.attn_ragged(lens, k, v, q, nH, nKV, hd, scale, softcap, kv="i8")
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))
    # and it is a different cache from the f16 one: the quantization is visible
    f16 = dev.attn_ragged(lens, k, v, q, nH, nKV, hd, scale, softcap)
    assert np.abs(got - f16).max() > 1e-4


def test_ragged_attention_i8_long_split(dev):
    lens = [1000, 4097, 128, 2050]
    nH, nKV, hd = 32, 8, 128
    tot, kvd = sum(lens), nKV * hd
    rng = np.random.default_rng(5)
    k = rng.standard_normal((tot, kvd), dtype=np.float32) * np.exp(rng.standard_normal((tot, 1), dtype=np.float32))  # rows of very different scale
    v = rng.standard_normal((tot, kvd), dtype=np.float32)
    q = rng.standard_normal((len(lens), nH * hd), dtype=np.float32)
    scale = float(1.0 / np.sqrt(hd))
    for softcap in (0.0, 50.0):
        got = dev.attn_ragged(lens, k, v, q, nH, nKV, hd, scale, softcap, kv="i8")
        want = oracle_attn(lens, i8_round_trip(k, nKV, hd), i8_round_trip(v, nKV, hd), q, nH, nKV, hd, scale, softcap)
        err = np.abs(got - want).max() / np.abs(want).max()
        assert err <= 1e-4, (softcap, err)


def rows_as_sequences(lens, nq, k, v):
    """The query rows of rd_attn_ragged_rows restated as one-row sequences: row j of sequence i sees keys 0..len-nq+j."""
    rl, ks, vs = [], [], []
    off = 0
    for n, m in zip(lens, nq):
        for j in range(m):
            see = n - m + 1 + j
            rl.append(see), ks.append(k[off:off + see]), vs.append(v[off:off + see])
        off += n
    return rl, np.concatenate(ks), np.concatenate(vs)


@pytest.mark.parametrize("kv", ["f16", "i8"])
@pytest.mark.parametrize("nH,nKV,hd", [(4, 1, 64), (8, 8, 128), (14, 2, 64), (32, 8, 128), (16, 2, 128)])
def test_rows_of_a_sequence_share_items_and_equal_solo_rows(dev, nH, nKV, hd, kv):
    """Several positions of one sequence in one item (they share every K and V read): each row against the oracle and
    bit-identical to the same row as a sequence of its own. The lengths put groups across a block boundary (where the rows
    part, their cuts differing), at a block's last key, past the split threshold, and past 128 blocks."""
    lens = [5, 64, 67, 130, 300, 1100, 1, 8300]
    nq = [5, 3, 6, 9, 2, 7, 1, 5]  # the last sequence is cut into more than 16 items: the combine folds them in rounds
    tot, kvd = sum(lens), nKV * hd
    k = synth.normal(11, tot * kvd).reshape(tot, kvd).astype(np.float16).astype(np.float32)  # exactly what the f16 cache holds
    v = synth.normal(12, tot * kvd).reshape(tot, kvd).astype(np.float16).astype(np.float32)
    q = synth.normal(13, sum(nq) * nH * hd).reshape(sum(nq), nH * hd)
    scale = float(1.0 / np.sqrt(hd))
    for softcap in (0.0, 30.0):
        got = dev.attn_ragged_rows(lens, nq, k, v, q, nH, nKV, hd, scale, softcap, kv=kv)
        rl, k1, v1 = rows_as_sequences(lens, nq, k, v)
        solo = dev.attn_ragged(rl, k1, v1, q, nH, nKV, hd, scale, softcap, kv=kv)
        assert np.array_equal(got.view(np.uint32), solo.view(np.uint32)), np.abs(got - solo).max()
        rt = (lambda x: x) if kv == "f16" else (lambda x: i8_round_trip(x, nKV, hd))
        want = oracle_attn(rl, rt(k1), rt(v1), q, nH, nKV, hd, scale, softcap)
        err = np.abs(got - want).max() / np.abs(want).max()
        assert err <= 1e-4, (softcap, err)


@pytest.mark.parametrize("kv", ["f16", "i8"])
def test_short_work_lists_run_two_units_in_flight_with_the_same_bits(dev, kv):
    """A work list of at most one item per SIMD runs the kernel that keeps two units of 32 keys in flight per wave; with the
    switch that turns it off the plain kernel runs. Same units in the same order: identical output bits."""
    import os
    lens = [1, 31, 32, 33, 64, 97, 700, 2049]
    nH, nKV, hd = 8, 2, 128
    tot, kvd = sum(lens), nKV * hd
    k = synth.normal(21, tot * kvd).reshape(tot, kvd)
    v = synth.normal(22, tot * kvd).reshape(tot, kvd)
    q = synth.normal(23, len(lens) * nH * hd).reshape(len(lens), nH * hd)
    scale = float(1.0 / np.sqrt(hd))
    for softcap in (0.0, 20.0):
        deep = dev.attn_ragged(lens, k, v, q, nH, nKV, hd, scale, softcap, kv=kv)
        os.environ["ROCMDECODE_NO_DEEP_ATTN"] = "1"
        try:
            plain = dev.attn_ragged(lens, k, v, q, nH, nKV, hd, scale, softcap, kv=kv)
        finally:
            del os.environ["ROCMDECODE_NO_DEEP_ATTN"]
        assert np.array_equal(deep.view(np.uint32), plain.view(np.uint32)), softcap


@pytest.mark.parametrize("kv", ["f16", "i8"])
def test_long_sequences_are_cut_into_more_than_sixteen_items(dev, kv):
    """Beyond 128 blocks an item stays at eight blocks, so the items of a (sequence, kv head) outnumber what the combine folds in
    one round: 8193 keys (17 items), 9000 (18) and 20000 (40) beside a short sequence, against the oracle."""
    lens = [8193, 9000, 300, 20000]
    nH, nKV, hd = 8, 2, 128
    tot, kvd = sum(lens), nKV * hd
    rng = np.random.default_rng(31)
    k = rng.standard_normal((tot, kvd), dtype=np.float32).astype(np.float16).astype(np.float32)
    v = rng.standard_normal((tot, kvd), dtype=np.float32).astype(np.float16).astype(np.float32)
    q = rng.standard_normal((len(lens), nH * hd), dtype=np.float32)
    scale = float(1.0 / np.sqrt(hd))
    got = dev.attn_ragged(lens, k, v, q, nH, nKV, hd, scale, 0.0, kv=kv)
    rt = (lambda x: x) if kv == "f16" else (lambda x: i8_round_trip(x, nKV, hd))
    want = oracle_attn(lens, rt(k), rt(v), q, nH, nKV, hd, scale, 0.0)
    err = np.abs(got - want).max() / np.abs(want).max()
    assert err <= 1e-4, err
    again = dev.attn_ragged(lens, k, v, q, nH, nKV, hd, scale, 0.0, kv=kv)
    assert np.array_equal(got.view(np.uint32), again.view(np.uint32))
