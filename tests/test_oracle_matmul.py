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
