"""GPU parity of the kernel-level entry points against the CPU oracle, through the C ABI.

Bars: Q4_K dequantization bit-exact; the activation quantizer's codes, scales and sums bit-exact; the int8-MFMA GEMMs
(Q4_K, int8, int4-g32) within 1e-5 of the f64 sum measured against the output's rms, the reference's own bar for its GPU
kernels (backend/cuda/kernels/actgroup_kernel_test.go:360): the dots are exact integers and only the f32 fold's order differs
from the oracle's. Every batched row equals the row computed alone, bit for bit.
"""
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


def rel_err(got, want):
    """max |got-want| over the rms of want: error relative to the typical output magnitude."""
    want = want.astype(np.float64)
    return float(np.abs(got.astype(np.float64) - want).max() / (np.sqrt((want * want).mean()) + 1e-30))


@pytest.mark.parametrize("N,K", [(32, 256), (96, 768), (200, 3072)])
def test_dequant_q4k_bit_exact(dev, N, K):
    rng = np.random.default_rng(N * K)
    raw = rng.integers(0, 256, N * (K // 256) * 144, dtype=np.uint8).reshape(-1, 144)
    # finite f16 d and dmin (exponent 5..11), as the reference's fixtures set them
    for off in (0, 2):
        h = (rng.integers(5, 12, len(raw)).astype(np.uint16) << 10) | rng.integers(0, 1024, len(raw)).astype(np.uint16)
        raw[:, off] = h & 0xFF
        raw[:, off + 1] = h >> 8
    raw[::5, 4:16] = 0xFF  # saturated scales and mins
    want = ob.dequant_q4k(raw).reshape(N, K)
    got = dev.dequant_q4k(raw, N, K)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequant_q4k_synth_bit_exact(dev):
    blocks = synth.q4k_normal(7, 128, 1024)
    want = ob.dequant_q4k(blocks).reshape(128, 1024)
    assert np.array_equal(dev.dequant_q4k(blocks, 128, 1024).view(np.uint32), want.view(np.uint32))
    assert abs(float(want.std()) - 0.02) < 2e-3


@pytest.mark.parametrize("M", [1, 4, 5, 32, 33, 64, 100, 128, 131])
@pytest.mark.parametrize("N,K", [(128, 256), (160, 1024), (512, 4096)])
def test_gemm_q4k(dev, M, N, K):
    blocks = synth.q4k_normal(11 + N, N, K)
    a = synth.normal(100 + M, M * K).reshape(M, K)
    w = ob.WMat(ob.OR_Q4K, N, K, blocks, act_group=32)
    want = ob.matmul(w, a)
    ref64 = ob.matmul_f64ref(w, a)
    got = dev.gemm_q4k(blocks, N, K, a)
    assert rel_err(want, ref64) < 1e-5  # the oracle itself, against the f64 sum (the reference's own kernel bar)
    assert rel_err(got, ref64) < 1e-5
    # batch invariance: a row computed in a batch equals the same row alone, bit for bit
    solo = dev.gemm_q4k(blocks, N, K, a[:1])
    assert np.array_equal(solo[0].view(np.uint32), got[0].view(np.uint32))


def test_gemm_q4k_rows_past_32_equal_solo_rows(dev):
    """More than 32 rows go through the kernel in passes of 32; every row must come out as it does alone, bit for bit."""
    N, K, M = 416, 2048, 131
    blocks = synth.q4k_normal(21, N, K)
    a = synth.normal(22, M * K).reshape(M, K)
    wide = dev.gemm_q4k(blocks, N, K, a)
    for r in (0, 31, 32, 77, 130):
        solo = dev.gemm_q4k(blocks, N, K, a[r:r + 1])
        assert np.array_equal(solo[0].view(np.uint32), wide[r].view(np.uint32))


@pytest.mark.parametrize("M,N,K", [(300, 160, 2048), (200, 256, 14336), (512, 4096, 768), (129, 6144, 4096)])
def test_gemm_q4k_many_row_kernel_equals_the_32_row_kernel(dev, M, N, K):
    """Past 32 rows four M-tiles share each decoded weight tile (one group of waves for a large grid, two for a small one, over
    one K range or several, one split or two): every row comes out as the 32-row kernel and the one-row kernel give it, bit for
    bit, and within 1e-5 of the f64 sum."""
    blocks = synth.q4k_normal(31 + N, N, K)
    a = synth.normal(32 + M, M * K).reshape(M, K)
    wide = dev.gemm_q4k(blocks, N, K, a)
    for r0 in (0, 96, M - 32):
        part = dev.gemm_q4k(blocks, N, K, a[r0:r0 + 32])
        assert np.array_equal(part.view(np.uint32), wide[r0:r0 + 32].view(np.uint32)), r0
    solo = dev.gemm_q4k(blocks, N, K, a[M - 1:M])
    assert np.array_equal(solo[0].view(np.uint32), wide[M - 1].view(np.uint32))
    rows = [0, 33, M - 1]
    w = ob.WMat(ob.OR_Q4K, N, K, blocks, act_group=32)
    assert rel_err(wide[rows], ob.matmul_f64ref(w, a[rows])) < 1e-5


def test_gemm_q4k_random_blocks_and_saturated_scales(dev):
    """Random bytes reach every code, scale and minimum (quantized normals do not), with every fifth block's 6-bit fields saturated:
    the shapes of the reference's own kernel test (actgroup_kernel_test.go:305-364, K = 3072, N = 200 rounded to whole tiles)."""
    N, K, M = 224, 3072, 5
    rng = np.random.default_rng(1)
    raw = rng.integers(0, 256, N * (K // 256) * 144, dtype=np.uint8).reshape(-1, 144)
    for off in (0, 2):
        h = (rng.integers(5, 12, len(raw)).astype(np.uint16) << 10) | rng.integers(0, 1024, len(raw)).astype(np.uint16)
        raw[:, off] = h & 0xFF
        raw[:, off + 1] = h >> 8
    raw[::5, 4:16] = 0xFF
    a = synth.normal(3, M * K).reshape(M, K)
    w = ob.WMat(ob.OR_Q4K, N, K, raw, act_group=32)
    got = dev.gemm_q4k(raw, N, K, a)
    assert rel_err(got, ob.matmul_f64ref(w, a)) < 1e-5
    # one row alone runs on the vector ALU, a batch on the matrix cores: the same bits on every code, scale and minimum
    for r in range(M):
        solo = dev.gemm_q4k(raw, N, K, a[r:r + 1])
        assert np.array_equal(solo[0].view(np.uint32), got[r].view(np.uint32)), r


def test_one_row_path_equals_batch_rows_at_the_step_shapes(dev):
    """The one-row kernels (v_dot4 on the vector ALU) against rows of a batch (int8 matrix cores), bit for bit, at shapes that take
    each plan of the step: four waves a tile in one split, eight waves in two K splits, activations from tiny to large, a zero row."""
    for N, K, seed in ((14336, 4096, 5), (4096, 14336, 6), (6144, 4096, 7)):
        blocks = synth.q4k_normal(seed, N, K)
        a = synth.normal(seed + 10, 6 * K).reshape(6, K)
        a[1] *= 1e-4
        a[2] *= 300.0
        a[3] = 0.0
        a[4, ::7] = 0.0
        wide = dev.gemm_q4k(blocks, N, K, a)
        for r in range(6):
            solo = dev.gemm_q4k(blocks, N, K, a[r:r + 1])
            assert np.array_equal(solo[0].view(np.uint32), wide[r].view(np.uint32)), (N, K, r)


@pytest.mark.parametrize("M,K", [(1, 32), (3, 256), (32, 4096), (40, 896), (7, 14336)])
def test_activation_quantizer_bits(dev, M, K):
    """rd_quant_act against the oracle's QuantizeActQ(group 32), which the reference's fingerprint pins: codes, scales and the
    scaled code sums the Q4_K minimum term multiplies, bit for bit, on normal rows, an all-zero group (scale 1, codes 0), values on
    exact half-way points between two codes (round half away from zero, where round-to-even differs) and a saturating outlier."""
    a = synth.normal(5 + M, M * K).reshape(M, K)
    a[0, :32] = 0.0  # an all-zero group
    if K >= 64:  # a group whose largest magnitude is 127 * 2^-3: x / scale is exact, and (c + 0.5) * scale is a tie between c and c+1
        g = a[M - 1, 32:64]
        c = np.random.default_rng(K).integers(-126, 126, 32).astype(np.float32)
        g[:] = (c + 0.5) * 0.125
        g[0] = 127 * 0.125
        g[1] = -127 * 0.125
    a[M // 2, K - 1] = 1e4  # an outlier: its group's other codes collapse to 0
    codes, scales, sums = dev.quant_act(a)
    q, S = ob.quantize_act(a, 32)
    assert np.array_equal(codes, q)
    assert np.array_equal(scales.view(np.uint32), S.view(np.uint32))
    want_sums = S * q.reshape(M, -1, 32).sum(-1).astype(np.float32)
    assert np.array_equal(sums.view(np.uint32), want_sums.view(np.uint32))
    if K >= 64:
        rne = np.clip(np.rint(a[M - 1, 32:64] / 0.125), -127, 127)
        assert (rne != q[M - 1, 32:64]).sum() >= 8  # the tie rows do tell half-away from round-to-even


def test_gemm_q4k_fused_gate_up(dev):
    N, K, M = 512, 1024, 9
    g, u = synth.q4k_normal(1, N, K, 0.05), synth.q4k_normal(2, N, K, 0.05)
    a = synth.normal(3, M * K).reshape(M, K)
    gate = ob.matmul(ob.WMat(ob.OR_Q4K, N, K, g, act_group=32), a)
    up = ob.matmul(ob.WMat(ob.OR_Q4K, N, K, u, act_group=32), a)
    want = ob.swiglu(gate, up)
    got = dev.gemm_q4k(g, N, K, a, blocks2=u)
    assert rel_err(got, want) < 1e-4  # silu(gate) * up of two GEMM outputs each within 1e-5


@pytest.mark.parametrize("M", [1, 9, 32, 40, 300])
def test_fused_gate_up_kernel(dev, M):
    """The decode step's single-launch gate|up + SwiGLU + quantization kernel, on its own."""
    from tests.test_gpu_baseline_shapes import check_fused
    I, K = 512, 1024
    g, u = synth.q4k_normal(1, I, K, 0.05), synth.q4k_normal(2, I, K, 0.05)
    a = synth.normal(3, M * K).reshape(M, K)
    gate = ob.matmul(ob.WMat(ob.OR_Q4K, I, K, g, act_group=32), a)
    up = ob.matmul(ob.WMat(ob.OR_Q4K, I, K, u, act_group=32), a)
    got = dev.gateup_q4k_quant(g, u, I, K, a)
    check_fused(got, gate, up)
    solo = dev.gateup_q4k_quant(g, u, I, K, a[:1])  # one row: the vector-ALU kernel; the same quantized activations, bit for bit
    assert np.array_equal(solo[0].view(np.uint32), got[0].view(np.uint32))


@pytest.mark.parametrize("M,N,K", [(1, 64, 128), (7, 256, 896), (32, 1024, 4096), (5, 96, 96)])
def test_gemm_w8a8(dev, M, N, K):
    q, s = synth.w8a8_normal(5, N, K)
    a = synth.normal(6, M * K).reshape(M, K)
    w = ob.WMat(ob.OR_W8A8, N, K, q, s, act_group=32)
    ref64 = ob.matmul_f64ref(w, a)
    got = dev.gemm_w8a8(q, s, a)
    assert rel_err(got, ref64) < 1e-5
    for r in range(min(M, 3)):  # a row alone (the vector-ALU kernel) is the row of the batch, bit for bit
        assert np.array_equal(dev.gemm_w8a8(q, s, a[r:r + 1])[0].view(np.uint32), got[r].view(np.uint32)), r


@pytest.mark.parametrize("M,N,K", [(1, 64, 128), (16, 768, 2048), (16, 2048, 768), (3, 64, 160)])
def test_gemm_w4a8(dev, M, N, K):
    nib, s16 = synth.w4a8_normal(8, N, K)
    a = synth.normal(9, M * K).reshape(M, K)
    w = ob.WMat(ob.OR_W4A8, N, K, nib, s16, act_group=32)
    ref64 = ob.matmul_f64ref(w, a)
    got = dev.gemm_w4a8(nib, s16, K, a)
    assert rel_err(got, ref64) < 1e-5
    for r in range(min(M, 3)):  # a row alone (the vector-ALU kernel) is the row of the batch, bit for bit
        assert np.array_equal(dev.gemm_w4a8(nib, s16, K, a[r:r + 1])[0].view(np.uint32), got[r].view(np.uint32)), r


@pytest.mark.parametrize("M,K", [(1, 32), (3, 256), (32, 4096), (40, 896), (7, 14336)])
def test_activation_quantizer_per_row_bits(dev, M, K):
    """rd_quant_act(act_group 0) against the oracle's QuantizeRowInt8 per row (fingerprint-pinned): codes and the row's one scale
    bit for bit, on normal rows, an all-zero row (scale 1, codes 0), a row of exact half-way points (round half away from zero)
    and a row with a saturating outlier."""
    a = synth.normal(15 + M, M * K).reshape(M, K)
    if M > 1:
        a[1] = 0.0  # an all-zero row
    g = a[M - 1]
    c = np.random.default_rng(K).integers(-126, 126, K).astype(np.float32)
    g[:] = (c + 0.5) * 0.125  # maxabs 127/8: x / scale is exact and (c + 0.5) * scale is a tie between c and c + 1
    g[0], g[1] = 127 * 0.125, -127 * 0.125
    if M > 2:
        a[M // 2, K - 1] = 1e4  # an outlier: the row's other codes collapse to 0
    codes, scales, _ = dev.quant_act(a, 0)
    q, S = ob.quantize_act(a, 0)
    assert np.array_equal(codes, q)
    assert np.array_equal(scales.view(np.uint32), S[:, 0].view(np.uint32))
    rne = np.clip(np.rint(g / 0.125), -127, 127)
    assert (rne != q[M - 1]).sum() >= K // 4  # the tie row does tell half-away from round-to-even


@pytest.mark.parametrize("M,N,K", [(1, 64, 128), (7, 256, 896), (32, 1024, 4096), (5, 96, 96), (131, 160, 2048), (4, 4096, 14336)])
def test_gemm_w8a8_per_row_bit_exact(dev, M, N, K):
    """int8 weights x per-row int8 activations (ActQuantGroup 0, the lane goinfer's staged QuantBackend.MatmulW8A8 hook serves):
    an exact int32 dot over the whole of K, then two rounded multiplies. The oracle's twin is digest-pinned to linalg.MatmulBTW8A8
    on all three reference configurations; the GPU equals it bit for bit, in a batch (matrix cores), alone (vector ALU) and past
    32 rows (further M-tiles)."""
    q, s = synth.w8a8_normal(5, N, K)
    a = synth.normal(6, M * K).reshape(M, K)
    a[0, : K // 2] *= 30.0
    want = ob.matmul(ob.WMat(ob.OR_W8A8, N, K, q, s, act_group=0), a)
    got = dev.gemm_w8a8(q, s, a, act_group=0)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    solo = dev.gemm_w8a8(q, s, a[M - 1:M], act_group=0)
    assert np.array_equal(solo[0].view(np.uint32), want[M - 1].view(np.uint32))


@pytest.mark.parametrize("M,N,K", [(1, 64, 128), (16, 768, 2048), (16, 2048, 768), (3, 64, 160), (40, 128, 4096)])
def test_gemm_w4a8_per_row(dev, M, N, K):
    """int4-g32 weights x per-row int8 activations (ActQuantGroup 0: the "int8 per-token activations" of the Qwen3-MoE benchmark configuration, the staged
    QuantBackend4.MatmulW4A8 hook and the experts' kernels): within 1e-5 of the f64 sum like every other lane (the reference's
    own kernel bar), the oracle too; a batched row is the row alone, bit for bit."""
    nib, s16 = synth.w4a8_normal(8, N, K)
    a = synth.normal(9, M * K).reshape(M, K)
    a[0, : K // 2] *= 30.0  # groups of very different magnitude: the per-32 lane would give another answer
    w = ob.WMat(ob.OR_W4A8, N, K, nib, s16, act_group=0)
    ref64 = ob.matmul_f64ref(w, a)
    got = dev.gemm_w4a8(nib, s16, K, a, act_group=0)
    assert rel_err(ob.matmul(w, a), ref64) < 1e-5
    assert rel_err(got, ref64) < 1e-5
    assert rel_err(dev.gemm_w4a8(nib, s16, K, a, act_group=32), ref64) > 1e-4  # not the per-32 lane by another name
    for r in range(min(M, 3)):
        assert np.array_equal(dev.gemm_w4a8(nib, s16, K, a[r:r + 1], act_group=0)[0].view(np.uint32), got[r].view(np.uint32)), r


def test_gemm_w4a8_per_row_random_nibbles(dev):
    """Random bytes reach every nibble value (quantized normals stop at +-7) and a wide range of scales."""
    N, K, M = 64, 1024, 5
    rng = np.random.default_rng(5)
    nib = rng.integers(0, 256, N * K // 2, dtype=np.uint8).reshape(N, K // 2)
    s16 = ((rng.integers(1, 20, N * (K // 32)).astype(np.uint16) << 10) | rng.integers(0, 1024, N * (K // 32)).astype(np.uint16)).reshape(N, K // 32)
    a = synth.normal(9, M * K).reshape(M, K)
    w = ob.WMat(ob.OR_W4A8, N, K, nib, s16, act_group=0)
    got = dev.gemm_w4a8(nib, s16, K, a, act_group=0)
    assert rel_err(got, ob.matmul_f64ref(w, a)) < 1e-5
    for r in range(M):
        assert np.array_equal(dev.gemm_w4a8(nib, s16, K, a[r:r + 1], act_group=0)[0].view(np.uint32), got[r].view(np.uint32)), r


def test_rmsnorm_rope_route(dev):
    x = synth.normal(1, 5 * 4096).reshape(5, 4096)
    w = synth.normal(2, 4096, 0.02, 1.0)
    got, want = dev.rmsnorm(x, w, 1e-5), ob.rmsnorm(x, w, 1e-5)
    assert np.abs(got - want).max() <= 1e-6 * np.abs(want).max()
    inv = 1.0 / (5e5 ** (np.arange(0, 128, 2) / 128.0))
    v = synth.normal(3, 3 * 4 * 128).reshape(3, 4 * 128)
    pos = [0, 17, 4095]
    got = dev.rope(v, 4, 128, pos, inv)
    assert np.array_equal(got[0], v[0])  # position 0 is the identity
    for r in range(3):
        want = ob.rope(v[r], 4, 128, pos[r], inv)
        assert np.abs(got[r] - want).max() <= 2e-6
    logits = synth.normal(4, 16 * 128).reshape(16, 128)
    logits[3, 7] = logits[3, 90]  # an exact tie: the lower index must win
    idx, wgt = dev.moe_route(logits, 8, True)
    for t in range(16):
        wi, ww = ob.route_experts(logits[t], 8, True)
        assert np.array_equal(idx[t], wi)
        assert np.array_equal(wgt[t].view(np.uint32), ww.view(np.uint32))


def test_issue_probes_run_and_decline_bad_arguments(dev):
    """The issue-rate probes (the int8 GEMMs' inner-loop instruction mix with every operand in registers) launch and time; the mix
    of all three parts takes at least as long as its longest part. Bad arguments are declined, not launched."""
    t = [float(np.median(dev.bench_kernel("issue", [mode, 2, 400], 1, 3))) for mode in range(4)]
    assert all(np.isfinite(x) and x > 0 for x in t), t
    assert t[3] > 0.9 * max(t[:3]), t
    for bad in ([4, 1, 100], [0, 3, 100], [0, 1, 0], [0, 1, 100, 5000]):
        with pytest.raises(capi.RocmError):
            dev.bench_kernel("issue", bad, 0, 1)
