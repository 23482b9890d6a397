"""The oracle's temperature-only sampler (Philox4x32-10 + Gumbel-max) against what the reference's own tests hold for it:
the Random123 known-answer vectors (internal/runtime/sampling/philox_test.go), the noise transform's closed form, range
and monotonicity (sampler_gumbel_test.go rule 4), the chi-square fit of the draw to softmax(l/T) under the reference's
pre-registered rule 1 (|z| < 4.5, bins under 20 expected merged), and its edge rows (rule 6 and TestGumbelDraw_edgeRows)."""
import numpy as np

from oracle import binding as ob

KAT = [  # counter[4], key[2] -> output[4]: Random123 kat_vectors "Philox4x32 10" as philox_test.go lists them
    ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0), (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
]


def test_philox_known_answers():
    for ctr, key, want in KAT:
        assert ob.philox4x32(ctr, key) == want


def test_noise_transform_and_range():
    assert 22.8 <= ob.gumbel_noise(0) <= 23.0
    assert -3.2 <= ob.gumbel_noise(0xFFFFFFFF) <= -3.0
    grid = (np.arange(100_000, dtype=np.uint64) * (1 << 32) // 100_000).astype(np.uint32)
    g = ob.gumbel_noise_many(grid)
    assert np.all(np.diff(g) <= 0)  # monotone non-increasing in h
    h = np.concatenate([grid, np.random.default_rng(4).integers(0, 1 << 32, 500_000, dtype=np.uint64).astype(np.uint32)])
    w = (h.astype(np.float64) + 0.5) / 4294967296.0
    ref = -np.log(-np.log1p(-w))
    assert np.abs(ob.gumbel_noise_many(h).astype(np.float64) - ref).max() <= 4e-6


def chi_square_z(counts, probs, n):
    exp = probs * n
    big = exp >= 20
    chi2 = float((((counts[big] - exp[big]) ** 2) / exp[big]).sum())
    bins = int(big.sum())
    if exp[~big].sum() >= 20:
        chi2 += float((counts[~big].sum() - exp[~big].sum()) ** 2 / exp[~big].sum())
        bins += 1
    df = bins - 1
    return (chi2 - df) / np.sqrt(2 * df)


def test_draw_fits_softmax():
    rng = np.random.default_rng(1)
    n = 400_000
    for T in (0.6, 1.0, 1.7):
        logits = (rng.standard_normal(40) * 2).astype(np.float32)
        ids = ob.gumbel_draw_many(logits, T, seed=7, draw0=0, count=n)
        p = np.exp((logits.astype(np.float64) - logits.max()) / T)
        p /= p.sum()
        z = chi_square_z(np.bincount(ids, minlength=40).astype(np.float64), p, n)
        assert abs(z) < 4.5, (T, z)


def test_draw_streams_and_edges():
    rng = np.random.default_rng(8)
    logits = (rng.standard_normal(5000) * 2).astype(np.float32)
    a = ob.gumbel_draw_many(logits, 0.9, 21, 0, 300)
    assert np.array_equal(a, ob.gumbel_draw_many(logits, 0.9, 21, 0, 300))
    assert (a == ob.gumbel_draw_many(logits, 0.9, 22, 0, 300)).sum() <= 150  # the seed reaches the generator
    assert np.array_equal(a[5:], ob.gumbel_draw_many(logits, 0.9, 21, 5, 295))  # draw i is a function of (seed, i) only
    assert a[3] == ob.gumbel_draw(logits, 0.9, 21, 3)
    # -Inf is never drawn; a fully masked row falls back to the argmax (index 0); flat logits draw uniformly
    l = np.full(64, -np.inf, np.float32)
    l[17], l[40] = 0.0, 0.5
    assert set(np.unique(ob.gumbel_draw_many(l, 1.0, 3, 0, 2000))) <= {17, 40}
    assert ob.gumbel_draw(np.full(64, -np.inf, np.float32), 1.0, 3, 0) == 0
    flat = ob.gumbel_draw_many(np.zeros(50, np.float32), 1.0, 9, 0, 300_000)
    assert abs(chi_square_z(np.bincount(flat, minlength=50).astype(np.float64), np.full(50, 0.02), 300_000)) < 4.5
    # an absurdly small temperature is the argmax, and a temperature <= 0 means 1 (Sampler.gumbelDraw's guards)
    assert ob.gumbel_draw(np.array([1, 9, 3], np.float32), 1e-40, 1, 0, guarded=True) == 1
    assert ob.gumbel_draw(logits, 0.0, 21, 3, guarded=True) == ob.gumbel_draw(logits, 1.0, 21, 3)
    # a lower temperature concentrates: at T -> small the draw is the argmax almost surely
    assert (ob.gumbel_draw_many(logits, 0.01, 5, 0, 200) == int(np.argmax(logits))).mean() > 0.9
