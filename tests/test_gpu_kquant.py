"""GPU parity of the Q5_K and Q6_K lanes against the CPU oracle, through the C ABI.

Bars as for Q4_K: dequantization bit-exact; GEMMs within 1e-5 of the f64 sum over the dequantized weights and the quantized
activations, measured against the output's rms (the reference's own kernel bar, backend/cuda/kernels/actgroup_kernel_test.go:360):
the codes are 5- and 6-bit integers, the dots exact int32 on the int8 matrix cores, only the f32 fold's order differs from the
oracle's; a row computed in a batch bit-identical to the row alone; a model whose projections mix Q4_K with
Q5_K / Q6_K tensors — also inside one fused q|k|v or gate|up group — within the decode bar against the oracle.
"""
import numpy as np
import pytest

from goinfer_amd import capi, synth
from oracle import binding as ob

from tests.models import Pair, dense_cfg
from tests.test_gpu_model import check

pytestmark = pytest.mark.gpu

FMT = {"q5k": (176, ob.OR_Q5K, ob.dequant_q5k), "q6k": (210, ob.OR_Q6K, ob.dequant_q6k)}


@pytest.fixture(scope="module")
def dev():
    d = capi.Device(0)
    yield d
    d.close()


def rel_err(got, want):
    want = want.astype(np.float64)
    return float(np.abs(got.astype(np.float64) - want).max() / (np.sqrt((want * want).mean()) + 1e-30))


def random_blocks(fmt, rng, n):
    """Random bytes with finite f16 super-scales, some blocks with saturated sub-block scales."""
    bb = FMT[fmt][0]
    raw = rng.integers(0, 256, n * bb, dtype=np.uint8).reshape(n, bb)
    for off in ((0, 2) if fmt == "q5k" else (208,)):
        h = (rng.integers(5, 12, n).astype(np.uint16) << 10) | rng.integers(0, 1024, n).astype(np.uint16)
        h |= (rng.integers(0, 2, n).astype(np.uint16) << 15) if fmt == "q6k" else 0
        raw[:, off] = h & 0xFF
        raw[:, off + 1] = h >> 8
    if fmt == "q5k":
        raw[::5, 4:16] = 0xFF
    else:
        raw[::5, 192:208] = 0x80  # scale -128
        raw[1::5, 192:208] = 0x7F
    return raw


@pytest.mark.parametrize("fmt", ["q5k", "q6k"])
@pytest.mark.parametrize("N,K", [(32, 256), (96, 768), (200, 3072)])
def test_dequant_bit_exact(dev, fmt, N, K):
    raw = random_blocks(fmt, np.random.default_rng(N * K), N * (K // 256))
    want = FMT[fmt][2](raw).reshape(N, K)
    got = dev.dequant_kquant(fmt, raw, N, K)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("fmt", ["q5k", "q6k"])
@pytest.mark.parametrize("M", [1, 5, 32, 33])
@pytest.mark.parametrize("N,K", [(128, 256), (160, 1024), (512, 4096)])
def test_gemm(dev, fmt, M, N, K):
    blocks = synth.kquant_normal(fmt, 11 + N, N, K)
    a = synth.normal(100 + M, M * K).reshape(M, K)
    w = ob.WMat(FMT[fmt][1], N, K, blocks, act_group=32)
    want = ob.matmul(w, a)
    ref64 = ob.matmul_f64ref(w, a)
    got = dev.gemm_kquant(fmt, blocks, N, K, a)
    assert rel_err(want, ref64) < 1e-5
    assert rel_err(got, ref64) < 1e-5
    solo = dev.gemm_kquant(fmt, blocks, N, K, a[:1])
    assert np.array_equal(solo[0].view(np.uint32), got[0].view(np.uint32))


@pytest.mark.parametrize("fmt", ["q5k", "q6k"])
@pytest.mark.parametrize("M,N,K", [(70, 160, 2048), (300, 256, 14336), (512, 4096, 768), (129, 6144, 1024)])
def test_gemm_many_rows_equal_the_32_row_kernel(dev, fmt, M, N, K):
    """From 65 rows a pass runs the many-row kernel (four M-tiles against each tile decoded once; one or two groups of waves by the
    size of the grid, one K range or several): every row is the row of the 32-row kernel, bit for bit, on random blocks (every code,
    sign and scale value), and within 1e-5 of the f64 sum."""
    raw = random_blocks(fmt, np.random.default_rng(7 + M), N * (K // 256))
    a = synth.normal(32 + M, M * K).reshape(M, K)
    wide = dev.gemm_kquant(fmt, raw, N, K, a)
    for r0 in (0, 64, M - 32):
        part = dev.gemm_kquant(fmt, raw, N, K, a[r0:r0 + 32])
        assert np.array_equal(part.view(np.uint32), wide[r0:r0 + 32].view(np.uint32)), r0
    rows = [0, 33, M - 1]
    w = ob.WMat(FMT[fmt][1], N, K, raw, act_group=32)
    assert rel_err(wide[rows], ob.matmul_f64ref(w, a[rows])) < 1e-5


@pytest.mark.parametrize("fmt", ["q5k", "q6k"])
def test_gemm_random_blocks(dev, fmt):
    """Every code, sign and scale value: random blocks rather than quantized normals."""
    N, K, M = 64, 512, 8
    raw = random_blocks(fmt, np.random.default_rng(5), N * (K // 256))
    a = synth.normal(77, M * K).reshape(M, K)
    w = ob.WMat(FMT[fmt][1], N, K, raw, act_group=32)
    ref64 = ob.matmul_f64ref(w, a)
    got = dev.gemm_kquant(fmt, raw, N, K, a)
    assert rel_err(got, ref64) < 1e-5
    for r in (0, M - 1):
        assert np.array_equal(dev.gemm_kquant(fmt, raw, N, K, a[r:r + 1])[0].view(np.uint32), got[r].view(np.uint32)), r


@pytest.mark.parametrize("kinds", [
    dict(o="q6k", down="q6k", head="q6k"),
    dict(q="q5k", k="q5k", v="q5k", gate="q5k", up="q5k", down="q5k"),
    dict(q="q6k", k="q6k", v="q6k", gate="q6k", up="q6k", o="q5k", head="q5k"),
    dict(v="q6k", down="q6k", head="q6k"),      # the GGUF Q4_K_M pattern: q, k, gate, up Q4_K; v, down, head Q6_K
    dict(v="w8a8", down="w8a8"),                # the same file as goinfer's q4k mode loads it: int8 copies of the Q6_K tensors
    dict(q="q5k", k="q5k", v="q6k", up="q6k"),  # Q5_K_M-like, and a gate|up pair that differs
], ids=["q6k-o-down-head", "q5k-fused", "q6k-fused-q5k-head", "q4km-mixed-qkv", "q4k-int8-mixed-qkv", "q5km-mixed-qkv-gateup"])
def test_model_mixed_kinds(dev, kinds):
    """Ragged batched decode, teacher-forced, against the oracle on the same blocks; batched rows == solo rows."""
    rng = np.random.default_rng(9)
    cfg = dense_cfg(n_layers=2, hidden=256, inter=512, vocab=512)
    check(Pair(cfg, seed=31, dev=dev, slots=8, kinds=kinds), [list(rng.integers(0, 512, n)) for n in (3, 40, 70)], steps=4)


@pytest.mark.parametrize("kinds", [dict(v="q6k", down="q6k", head="q6k"), dict(q="q5k", k="q5k", v="q6k", up="q6k", o="q5k")], ids=["q4km", "q5km"])
def test_mixed_kinds_prompt_pass_equals_token_by_token(dev, kinds):
    """A 150-row prompt pass over a model whose projections mix Q4_K, Q5_K and Q6_K (each tensor through its own many-row kernel):
    the last row's logits and the KV left behind are the token-by-token path's, bit for bit."""
    cfg = dense_cfg(n_layers=2, hidden=512, n_heads=8, n_kv=2, head_dim=64, inter=1024, vocab=512)
    pair = Pair(cfg, seed=33, dev=dev, slots=2, ctx_cap=160, kinds=kinds)
    try:
        toks = list(np.random.default_rng(3).integers(0, cfg["vocab"], 150))
        got = pair.gpu.prefill_last(0, 0, pair.emb[toks])
        want = np.stack([pair.gpu.forward(1, p, pair.emb[t]) for p, t in enumerate(toks)])[-1]
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        for layer in range(cfg["n_layers"]):
            ka, va = pair.gpu.kv_download(0, layer, 0, 150)
            kb, vb = pair.gpu.kv_download(1, layer, 0, 150)
            assert np.array_equal(ka.view(np.uint32), kb.view(np.uint32)) and np.array_equal(va.view(np.uint32), vb.view(np.uint32)), layer
    finally:
        pair.close()
