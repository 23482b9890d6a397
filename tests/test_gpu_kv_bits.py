"""What the KV cache holds, bit for bit, on inputs that tell the rounding modes apart.

goinfer's f16 cache narrows with round-half-up on the dropped bits (internal/runtime/f16/f16.go:14-43, pinned in the oracle by the
linalg.F32ToF16 fingerprint); the int8 cache rounds code = x/scale half away from zero (linalg.QuantizeRowInt8 fingerprint). The
values here sit exactly half-way between two neighbours, where round-to-nearest-even and the reference's modes give different
bits, so a store that rounded the hardware's way fails. Both store paths are covered: rows the host uploads (UploadKV) and rows the
step's q|k|v epilogue writes, read back through rd_kv_download / rd_qkv_rope_store.
"""
import numpy as np
import pytest

from goinfer_amd import capi
from oracle import binding as ob
from tests.models import Pair, dense_cfg
from tests.util import inv_freq

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = capi.Device(0)
    yield d
    d.close()


def f16_tie_values(n, seed):
    """f32 values whose 13 dropped mantissa bits are exactly the half-way pattern (or one ulp to either side of it), over the
    binary16 normal range, the subnormal range, the carry into the next exponent, and both signs."""
    rng = np.random.default_rng(seed)
    exp = rng.integers(127 - 24, 127 + 15, n).astype(np.uint32)  # below 2^-14 the result is a binary16 subnormal
    top = rng.integers(0, 1024, n).astype(np.uint32)
    top[::7] = 0x3FF  # a round-up here carries into the exponent
    low = np.full(n, 0x1000, np.uint32)
    low[1::5] = 0x0FFF
    low[2::5] = 0x1001
    sign = rng.integers(0, 2, n).astype(np.uint32) << 31
    bits = sign | (exp << 23) | (top << 13) | low
    # in the subnormal range the half-way point moves up with the shift: make those exact ties as well
    sub = exp < 127 - 14
    sh = (127 - 14 - exp[sub]).astype(np.uint32)  # extra bits dropped
    m = (top[sub] << 13) | 0x800000
    drop = 13 + sh
    m = (m >> drop << drop) | (np.uint32(1) << (drop - 1))
    bits[sub] = sign[sub] | (exp[sub] << 23) | (m & 0x7FFFFF)
    return bits.view(np.float32)


def rne_round_trip(x):
    return x.astype(np.float16).astype(np.float32)


def test_uploaded_rows_are_narrowed_half_up(dev):
    cfg = dense_cfg(n_layers=1, hidden=256, n_heads=4, n_kv=2, head_dim=128, inter=256, vocab=256)
    pair = Pair(cfg, seed=3, dev=dev, slots=2, ctx_cap=256)
    try:
        n, kvd = 200, 2 * 128
        k = f16_tie_values(n * kvd, 1).reshape(n, kvd)
        v = f16_tie_values(n * kvd, 2).reshape(n, kvd)
        pair.gpu.kv_upload(1, 0, 0, k, v)
        gk, gv = pair.gpu.kv_download(1, 0, 0, n)
        wk, wv = ob.f16_round_trip(k), ob.f16_round_trip(v)
        assert (wk.view(np.uint32) != rne_round_trip(k).view(np.uint32)).mean() > 0.2  # the inputs do tell the two modes apart
        assert np.array_equal(gk.view(np.uint32), wk.view(np.uint32))
        assert np.array_equal(gv.view(np.uint32), wv.view(np.uint32))
    finally:
        pair.close()


@pytest.mark.parametrize("hd", [64, 128])
def test_step_epilogue_stores_half_up(dev, hd):
    """Position 0 rotates by the identity, so the stored K row is the narrowed projection row itself, bit for bit; V is never rotated."""
    nH, nKV, rows = 4, 2, 7
    inv = inv_freq(hd, 5e5)
    x = f16_tie_values(rows * (nH + 2 * nKV) * hd, 5).reshape(rows, -1)
    pos = np.array([0, 0, 0, 0, 0, 0, 0], np.int32)
    q, k, v = dev.qkv_rope_store(x, pos, nH, nKV, hd, inv)
    qd, kvd = nH * hd, nKV * hd
    assert np.array_equal(q.view(np.uint32), x[:, :qd].view(np.uint32))  # q stays f32
    wk, wv = ob.f16_round_trip(x[:, qd:qd + kvd]), ob.f16_round_trip(x[:, qd + kvd:])
    assert (wk.view(np.uint32) != rne_round_trip(x[:, qd:qd + kvd]).view(np.uint32)).mean() > 0.2
    assert np.array_equal(k.view(np.uint32), wk.view(np.uint32))
    assert np.array_equal(v.view(np.uint32), wv.view(np.uint32))
    # V at other positions too (K there is rotated: compared with the oracle's rope to f32 accuracy, then narrowed)
    pos = np.array([1, 63, 64, 65, 200, 4095, 17], np.int32)
    q, k, v = dev.qkv_rope_store(x, pos, nH, nKV, hd, inv)
    assert np.array_equal(v.view(np.uint32), wv.view(np.uint32))
    for r in range(rows):
        want = ob.rope(x[r, qd:qd + kvd], nKV, hd, int(pos[r]), inv)
        ref = ob.f16_round_trip(want)
        ulp = np.maximum(np.abs(ref) * 2.0 ** -10, 2.0 ** -24)
        assert (np.abs(k[r] - ref) <= ulp).all()  # the rotated value may sit across a rounding boundary from the oracle's: one f16 ulp
        assert (k[r].view(np.uint32) == ref.view(np.uint32)).mean() > 0.98


def int8_tie_rows(rows, nKV, hd, seed):
    """Heads whose largest magnitude is 127 * 2^e, so the scale is the power of two 2^e exactly and x/scale is exact: values at
    (c + 0.5) * 2^e are exact ties between the codes c and c+1."""
    rng = np.random.default_rng(seed)
    x = np.empty((rows, nKV, hd), np.float32)
    for r in range(rows):
        for h in range(nKV):
            e = float(2.0 ** int(rng.integers(-6, 5)))
            c = rng.integers(-127, 127, hd).astype(np.float32)
            frac = rng.choice(np.array([0.5, 0.5, 0.5, 0.25, 0.75, 0.0], np.float32), hd)
            vals = (c + frac) * e
            vals[int(rng.integers(0, hd))] = (127.0 if rng.integers(0, 2) else -127.0) * e
            x[r, h] = vals
    x[0, 0] = 0.0  # an all-zero head: scale 1, codes 0
    return x.reshape(rows, nKV * hd)


def oracle_int8_round_trip(x, nKV, hd):
    q, s = ob.quantize_rows_int8(x.reshape(-1, hd))
    return ob.dequantize_rows_int8(q, s).reshape(x.shape), q.reshape(x.shape), s


def test_int8_cache_rounds_half_away(dev):
    cfg = dense_cfg(n_layers=1, hidden=256, n_heads=4, n_kv=2, head_dim=128, inter=256, vocab=256)
    pair = Pair(cfg, seed=3, dev=dev, slots=2, ctx_cap=256, kv="i8")
    try:
        n, nKV, hd = 150, 2, 128
        k, v = int8_tie_rows(n, nKV, hd, 1), int8_tie_rows(n, nKV, hd, 2)
        pair.gpu.kv_upload(0, 0, 0, k, v)
        gk, gv = pair.gpu.kv_download(0, 0, 0, n)
        wk, qk, _ = oracle_int8_round_trip(k, nKV, hd)
        wv, _, _ = oracle_int8_round_trip(v, nKV, hd)
        rne = np.clip(np.rint(k.reshape(-1, hd) / (np.abs(k.reshape(-1, hd)).max(axis=1, keepdims=True) / 127 + 1e-30)), -127, 127)
        assert (rne.reshape(qk.shape) != qk).mean() > 0.1  # round-to-even codes would differ on these inputs
        assert np.array_equal(gk.view(np.uint32), wk.view(np.uint32))
        assert np.array_equal(gv.view(np.uint32), wv.view(np.uint32))
    finally:
        pair.close()


def test_step_epilogue_int8_store_rounds_half_away(dev):
    nH, nKV, hd, rows = 4, 2, 128, 9
    inv = inv_freq(hd, 1e6)
    kv = int8_tie_rows(rows, 2 * nKV, hd, 7)  # k heads then v heads
    x = np.concatenate([np.zeros((rows, nH * hd), np.float32), kv], axis=1)
    q, k, v = dev.qkv_rope_store(x, np.zeros(rows, np.int32), nH, nKV, hd, inv, kv="i8")
    wk, _, _ = oracle_int8_round_trip(kv[:, :nKV * hd], nKV, hd)
    wv, _, _ = oracle_int8_round_trip(kv[:, nKV * hd:], nKV, hd)
    assert np.array_equal(k.view(np.uint32), wk.view(np.uint32))
    assert np.array_equal(v.view(np.uint32), wv.view(np.uint32))


def test_kv_upload_with_many_kv_heads(dev):
    """An MHA shape whose kv width (32 heads x 128) is four times a block's thread limit: UploadKV must still serve it."""
    cfg = dense_cfg(n_layers=1, hidden=4096, n_heads=32, n_kv=32, head_dim=128, inter=256, vocab=256)
    pair = Pair(cfg, seed=5, dev=dev, slots=1, ctx_cap=128)
    try:
        n, kvd = 70, 32 * 128
        rng = np.random.default_rng(0)
        k, v = rng.standard_normal((n, kvd), dtype=np.float32), rng.standard_normal((n, kvd), dtype=np.float32)
        pair.gpu.kv_upload(0, 0, 0, k, v)
        gk, gv = pair.gpu.kv_download(0, 0, 0, n)
        assert np.array_equal(gk, ob.f16_round_trip(k)) and np.array_equal(gv, ob.f16_round_trip(v))
    finally:
        pair.close()


def test_kv_configure_needs_a_finalized_model(dev):
    cfg = dense_cfg(n_layers=1)
    m = capi.Model(dev, cfg, inv_freq(cfg["head_dim"], cfg["theta"]))
    try:
        with pytest.raises(capi.RocmError, match="finalize"):
            m.kv_configure(2, 128)
    finally:
        m.close()
