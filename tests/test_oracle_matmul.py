"""The oracle's k-quant matmul lanes against what the mathematics fixes, from pieces that are pinned on their own.

The weight dequantizers (Q4_K, Q5_K, Q6_K) and the activation quantizer are held bit-exact to the reference's fingerprints
(test_oracle_fingerprints.py). A matmul lane is then fixed up to f32 rounding: dst[m][n] = sum_k w[n][k] * (code[m][k] *
scale[m][k/32]). Each lane is checked against that sum formed in f64 by numpy from the pinned pieces, to 1e-5 of the output's
rms (the reference's own kernel bar, backend/cuda/kernels/actgroup_kernel_test.go:360). A dropped -dmin*m term, a wrong
sub-block scale index, the -32 centring or a misplaced high bit each fail it by orders of magnitude.
"""
import numpy as np
import pytest

from goinfer_amd import synth
from oracle import binding as ob

KINDS = {
    "q4k": (ob.OR_Q4K, lambda s, N, K: synth.q4k_normal(s, N, K), ob.dequant_q4k),
    "q5k": (ob.OR_Q5K, lambda s, N, K: synth.kquant_normal("q5k", s, N, K), ob.dequant_q5k),
    "q6k": (ob.OR_Q6K, lambda s, N, K: synth.kquant_normal("q6k", s, N, K), ob.dequant_q6k),
}


@pytest.mark.parametrize("fmt", sorted(KINDS))
@pytest.mark.parametrize("M,N,K", [(1, 32, 256), (5, 96, 1024), (32, 64, 2048)])
def test_kquant_matmul_is_the_sum_of_pinned_pieces(fmt, M, N, K):
    kind, make, dequant = KINDS[fmt]
    blocks = make(17 + N, N, K)
    a = synth.normal(5 + M, M * K).reshape(M, K)
    got = ob.matmul(ob.WMat(kind, N, K, blocks, act_group=32), a)
    w = dequant(blocks).reshape(N, K).astype(np.float64)
    q, S = ob.quantize_act(a, 32)
    aq = q.astype(np.float64) * np.repeat(S.astype(np.float64), 32, axis=1)
    want = aq @ w.T
    err = np.abs(got - want).max() / np.sqrt((want * want).mean())
    assert err < 1e-5, err
    # and the lane's own f64 twin used by the GPU tests agrees with the same sum
    ref = ob.matmul_f64ref(ob.WMat(kind, N, K, blocks, act_group=32), a)
    assert np.abs(ref - want).max() / np.sqrt((want * want).mean()) < 1e-6


@pytest.mark.parametrize("fmt", ["q5k", "q6k"])
def test_kquant_matmul_random_blocks(fmt):
    """Random bytes reach every code, fifth/high bit, scale and sign, which quantized normals do not."""
    kind, _, dequant = KINDS[fmt]
    bb = 176 if fmt == "q5k" else 210
    N, K, M = 32, 512, 3
    rng = np.random.default_rng(3)
    raw = rng.integers(0, 256, N * (K // 256) * bb, dtype=np.uint8).reshape(-1, bb)
    for off in ((0, 2) if fmt == "q5k" else (208,)):
        raw[:, off + 1] = 0x10 | (raw[:, off + 1] & 0x83 if fmt == "q6k" else raw[:, off + 1] & 3)  # small finite f16
    a = synth.normal(9, M * K).reshape(M, K)
    got = ob.matmul(ob.WMat(kind, N, K, raw, act_group=32), a)
    w = dequant(raw).reshape(N, K).astype(np.float64)
    q, S = ob.quantize_act(a, 32)
    want = (q.astype(np.float64) * np.repeat(S.astype(np.float64), 32, axis=1)) @ w.T
    assert np.abs(got - want).max() / np.sqrt((want * want).mean()) < 1e-5


def f16_bits_to_f64(bits):
    """binary16 bit patterns widened by numpy's own IEEE conversion (no oracle code involved)."""
    return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(np.float64)


def int4_weights_f64(nib, s16, N, K):
    """Canonical int4 rows as the reference states them (backend/cuda/kernels/actgroup_kernel_test.go:252-261: element k sits in
    nibble k%2 of byte k/2, low nibble first, value nib-8; backend/cuda/internal/wpack/wpack.go:165-207 is the permuted device
    form of the same words), times the binary16 group scale of k/32."""
    nib = np.asarray(nib, dtype=np.uint8).reshape(N, (K + 1) // 2)
    codes = np.empty((N, K), np.float64)
    codes[:, 0::2] = (nib & 15).astype(np.float64)[:, :(K + 1) // 2]
    codes[:, 1::2] = (nib >> 4).astype(np.float64)[:, :K // 2]
    scales = f16_bits_to_f64(np.asarray(s16).reshape(N, -1))
    return (codes - 8.0) * np.repeat(scales, 32, axis=1)[:, :K]


@pytest.mark.parametrize("M,N,K", [(1, 32, 128), (5, 96, 768), (16, 64, 2048), (3, 40, 96)])
def test_w4a8_matmul_is_the_sum_of_pinned_pieces(M, N, K):
    """The int4 lane (the MoE experts' kind) from pieces pinned on their own: quantize_int4's nibbles and binary16 scales
    (fingerprints QuantizeGroupInt4Row / QuantizeInt4 / F32ToF16) and quantize_act's codes and scales (QuantizeActQ). A wrong
    nibble order, a missing -8, a scale taken from the wrong group or widened wrongly fails by orders of magnitude."""
    w = synth.normal(31 + N, N * K, 0.02).reshape(N, K)
    nib, s16 = ob.quantize_int4(w)
    a = synth.normal(7 + M, M * K).reshape(M, K)
    mat = ob.WMat(ob.OR_W4A8, N, K, nib, s16, act_group=32)
    got = ob.matmul(mat, a)
    wd = int4_weights_f64(nib, s16, N, K)
    assert np.abs(wd - w).max() < 0.02 * 4.5 / 7 * 0.6  # and the pieces are a quantization of w at all
    q, S = ob.quantize_act(a, 32)
    want = (q.astype(np.float64) * np.repeat(S.astype(np.float64), 32, axis=1)) @ wd.T
    rms = np.sqrt((want * want).mean())
    assert np.abs(got - want).max() / rms < 1e-5
    assert np.abs(ob.matmul_f64ref(mat, a) - want).max() / rms < 1e-6


def test_w4a8_matmul_random_nibbles_and_scales():
    """Random bytes reach every nibble value and the scales' whole exponent range in use, which quantized normals do not."""
    N, K, M = 32, 512, 3
    rng = np.random.default_rng(5)
    nib = rng.integers(0, 256, N * K // 2, dtype=np.uint8).reshape(N, K // 2)
    s16 = ((rng.integers(1, 20, N * (K // 32)).astype(np.uint16) << 10) | rng.integers(0, 1024, N * (K // 32)).astype(np.uint16)).reshape(N, K // 32)
    a = synth.normal(9, M * K).reshape(M, K)
    mat = ob.WMat(ob.OR_W4A8, N, K, nib, s16, act_group=32)
    q, S = ob.quantize_act(a, 32)
    want = (q.astype(np.float64) * np.repeat(S.astype(np.float64), 32, axis=1)) @ int4_weights_f64(nib, s16, N, K).T
    rms = np.sqrt((want * want).mean())
    assert np.abs(ob.matmul(mat, a) - want).max() / rms < 1e-5
    assert np.abs(ob.matmul_f64ref(mat, a) - want).max() / rms < 1e-6


@pytest.mark.parametrize("M,N,K", [(1, 32, 128), (7, 64, 896), (32, 96, 4096)])
def test_w8a8_per32_matmul_is_the_sum_of_pinned_pieces(M, N, K):
    """The int8 lane with per-32 activations (LM head and the projections whose K is no multiple of 256), against the same sum:
    quantize_rows_int8's codes and per-row scales are pinned by QuantizeRowInt8, the activations by QuantizeActQ."""
    w = synth.normal(41 + N, N * K, 0.02).reshape(N, K)
    wq, ws = ob.quantize_rows_int8(w)
    a = synth.normal(3 + M, M * K).reshape(M, K)
    mat = ob.WMat(ob.OR_W8A8, N, K, wq, ws, act_group=32)
    q, S = ob.quantize_act(a, 32)
    wd = wq.astype(np.float64) * ws.astype(np.float64)[:, None]
    want = (q.astype(np.float64) * np.repeat(S.astype(np.float64), 32, axis=1)) @ wd.T
    rms = np.sqrt((want * want).mean())
    assert np.abs(ob.matmul(mat, a) - want).max() / rms < 1e-5
    assert np.abs(ob.matmul_f64ref(mat, a) - want).max() / rms < 1e-6


@pytest.mark.parametrize("M,N,K", [(1, 32, 128), (5, 96, 768), (16, 64, 2048), (3, 40, 96)])
def test_w4a8_per_row_matmul_is_the_sum_of_pinned_pieces(M, N, K):
    """The int4 lane with ONE activation scale per row (goinfer's ActQuantGroup 0: the experts' kernels and the staged MatmulW4A8
    hook, decoder/weightmat.go:909-912, backend/cuda/moe_rows.cu:24-106), from the same pinned pieces: the activations are
    quantize_act(group 0) = QuantizeRowInt8 per row. A per-group scale used where the row's belongs, or the row scale applied per
    group, moves the result by per cent, not 1e-5."""
    w = synth.normal(31 + N, N * K, 0.02).reshape(N, K)
    nib, s16 = ob.quantize_int4(w)
    a = synth.normal(7 + M, M * K).reshape(M, K)
    a[0, : K // 2] *= 40.0  # a row whose groups differ widely in magnitude: per-row and per-32 scales then differ by far
    mat = ob.WMat(ob.OR_W4A8, N, K, nib, s16, act_group=0)
    q, S = ob.quantize_act(a, 0)
    assert S.shape == (M, 1)
    want = (q.astype(np.float64) * S.astype(np.float64)) @ int4_weights_f64(nib, s16, N, K).T
    rms = np.sqrt((want * want).mean())
    assert np.abs(ob.matmul(mat, a) - want).max() / rms < 1e-5
    assert np.abs(ob.matmul_f64ref(mat, a) - want).max() / rms < 1e-6
    per32 = ob.matmul(ob.WMat(ob.OR_W4A8, N, K, nib, s16, act_group=32), a)
    assert np.abs(per32 - want).max() / rms > 1e-3  # the two lanes are different functions of the same inputs


def test_w4a8_per_row_random_nibbles_and_scales():
    N, K, M = 32, 512, 3
    rng = np.random.default_rng(6)
    nib = rng.integers(0, 256, N * K // 2, dtype=np.uint8).reshape(N, K // 2)
    s16 = ((rng.integers(1, 20, N * (K // 32)).astype(np.uint16) << 10) | rng.integers(0, 1024, N * (K // 32)).astype(np.uint16)).reshape(N, K // 32)
    a = synth.normal(9, M * K).reshape(M, K)
    mat = ob.WMat(ob.OR_W4A8, N, K, nib, s16, act_group=0)
    q, S = ob.quantize_act(a, 0)
    want = (q.astype(np.float64) * S.astype(np.float64)) @ int4_weights_f64(nib, s16, N, K).T
    rms = np.sqrt((want * want).mean())
    assert np.abs(ob.matmul(mat, a) - want).max() / rms < 1e-5
    assert np.abs(ob.matmul_f64ref(mat, a) - want).max() / rms < 1e-6


@pytest.mark.parametrize("M,N,K", [(1, 32, 128), (7, 64, 896), (32, 96, 4096)])
def test_w8a8_per_row_matmul_is_exact_in_integers(M, N, K):
    """The int8 lane with per-row activations is digest-pinned (linalg.MatmulBTW8A8, test_oracle_fingerprints.py). Independently:
    its value is f32(f32(f32(idot) * aS) * wS) with an exact integer dot, which numpy restates in int64 and float32."""
    w = synth.normal(41 + N, N * K, 0.02).reshape(N, K)
    wq, ws = ob.quantize_rows_int8(w)
    a = synth.normal(3 + M, M * K).reshape(M, K)
    q, S = ob.quantize_act(a, 0)
    idot = q.astype(np.int64) @ wq.astype(np.int64).T
    want = (idot.astype(np.float32) * S.astype(np.float32)) * ws.astype(np.float32)[None, :]
    got = ob.matmul(ob.WMat(ob.OR_W8A8, N, K, wq, ws, act_group=0), a)
    assert np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32))
