"""Pins the position -> entry map of the oracles: two independent implementations agree, every
random bit is used exactly once, the reference's parity property holds, and the Box-Muller
restatement matches a float64 math-library evaluation."""
import math

import numpy as np
import pytest

from oracle import jl_oracle as npo

R, G = npo.RADEMACHER, npo.NORMAL


@pytest.mark.parametrize("proj_type", [R, G])
@pytest.mark.parametrize(
    "seed,tiles,P,f0,nf,c0,nc",
    [
        (0, 256, 1000, 0, 1000, 0, 8),          # tile size 4: 250 used tiles
        (42, 256, 1_048_576, 4090, 300, 500, 12),   # crosses a tile boundary (tile size 4096)
        (7, 108, 10_241, 9_900, 341, 2040, 8),      # odd P, last tile is short
        (123, 4, 1000, 0, 1000, 3, 5),              # few tiles: many blocks per stream
        (2**32 - 1, 256, 25, 0, 25, 0, 16),         # P < tiles
    ],
)
def test_c_and_numpy_oracles_agree(c_oracle, proj_type, seed, tiles, P, f0, nf, c0, nc):
    a = c_oracle.materialize(seed, tiles, P, f0, nf, c0, nc, proj_type)
    b = npo.materialize(seed, tiles, P, f0, nf, c0, nc, proj_type)
    assert a.dtype == np.float32 and a.shape == (nf, nc)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_rademacher_uses_every_bit_of_a_block_once(c_oracle):
    # one tile of 128 features: entry j must be a distinct bit of the block's 128 bits
    seed, col = 99, 17
    P = 128
    words = c_oracle.philox([0, c_oracle.stream_name(seed, col, 0), 0, 0], [seed, 0])
    col_vals = c_oracle.materialize(seed, 1, P, 0, P, col, 1, R)[:, 0]
    # entry j is bit j of the block read as one 128-bit little-endian number
    block = sum(w << (32 * i) for i, w in enumerate(words))
    for j in range(128):
        assert col_vals[j] == (1.0 if (block >> j) & 1 else -1.0)
    # the second block of the stream serves features 128..255
    words1 = c_oracle.philox([1, c_oracle.stream_name(seed, col, 0), 0, 0], [seed, 0])
    block1 = sum(w << (32 * i) for i, w in enumerate(words1))
    col_vals = c_oracle.materialize(seed, 1, 256, 128, 128, col, 1, R)[:, 0]
    assert [v > 0 for v in col_vals] == [bool((block1 >> j) & 1) for j in range(128)]


def test_rademacher_values_and_balance(c_oracle):
    S = c_oracle.materialize(5, 256, 200_000, 0, 20_000, 0, 64, R)
    assert set(np.unique(S).tolist()) == {-1.0, 1.0}
    # 1.28M fair bits: |mean| < 5 sigma
    assert abs(S.mean()) < 5 / math.sqrt(S.size)
    # columns are different streams: correlation between neighbours is noise
    c = np.corrcoef(S[:, :16].T)
    assert np.abs(c - np.eye(16)).max() < 6 / math.sqrt(S.shape[0])
    # rows (features) too
    r = np.corrcoef(S[:64, :])
    assert np.abs(r - np.eye(64)).max() < 0.7


def test_streams_differ_across_tiles_columns_and_seeds(c_oracle):
    a = c_oracle.materialize(1, 256, 1 << 16, 0, 256, 0, 4, R)
    b = c_oracle.materialize(1, 256, 1 << 16, 256, 256, 0, 4, R)   # next tile (tile size 256)
    c = c_oracle.materialize(2, 256, 1 << 16, 0, 256, 0, 4, R)
    assert not np.array_equal(a, b) and not np.array_equal(a, c)
    assert not np.array_equal(a[:, 0], a[:, 1])
    # seed enters additively with the column and tile strides (fast_jl/random.cuh:15-17):
    # seed + 658105236 at column 0 has the stream name of (seed, column 1), but the seed is also
    # the generator's key: another projector seed never replays a stream of this one
    d = c_oracle.materialize((1 + 658105236) % 2**32, 256, 1 << 16, 0, 256, 0, 1, R)
    assert c_oracle.stream_name((1 + 658105236) % 2**32, 0, 0) == c_oracle.stream_name(1, 1, 0)
    assert not np.array_equal(d[:, 0], a[:, 1])


@pytest.mark.parametrize("P,expect_odd", [(10_240, False), (10_241, True)])
def test_parity_of_all_ones_projection(c_oracle, P, expect_odd):
    # tests/test_rademacher.py:65-108: all-ones input, every output has the parity of P
    G32 = np.ones((8, P), dtype=np.float32)
    out = c_oracle.project(G32, 64 if not expect_odd else 78, 256, 0, 24, R)
    assert np.all(out == np.round(out))
    assert np.all((out.astype(np.int64) % 2 == 1) == expect_odd)


def test_project_matches_numpy_matmul(c_oracle):
    rng = np.random.default_rng(3)
    for proj_type in (R, G):
        Gm = rng.standard_normal((5, 3000)).astype(np.float32)
        S = npo.materialize(11, 16, 3000, 0, 3000, 32, 10, proj_type).astype(np.float64)
        want = Gm.astype(np.float64) @ S
        got = c_oracle.project(Gm, 11, 16, 32, 10, proj_type)
        np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
        got2 = npo.project_fp64(Gm, 11, 16, np.arange(32, 42), proj_type)
        np.testing.assert_allclose(got2, want, rtol=1e-12, atol=1e-12)


def _ulp16(v):
    """Spacing of fp16 numbers at |v| (subnormal spacing below 2^-14)."""
    e = np.floor(np.log2(np.maximum(np.abs(v), 2.0**-14)))
    return 2.0 ** (e - 10)


def test_factor_tables_against_float64_math(c_oracle):
    # The tables of the normal entries are fp16 roundings of binary32 evaluations of
    # sqrt(-2 ln u), cos and sin.  A correctly rounded table computed with the float64 math
    # library can differ only where the exact value sits within the binary32 error (a few 2^-24)
    # of an fp16 rounding boundary: never by more than one fp16 step, and only rarely at all.
    R, C, S = npo.normal_tables()
    n = 1 << 14
    assert R.dtype == np.float16 and R.shape == C.shape == S.shape == (n,)
    x = np.arange(n, dtype=np.float64)
    want_r = np.sqrt(-2.0 * np.log((x + 0.5) / n))
    theta = (np.arange(n, dtype=np.float64) + 0.5) * (2 * np.pi) / n      # around the whole circle
    for got, want in ((R, want_r), (C, np.cos(theta)), (S, np.sin(theta))):
        got64 = got.astype(np.float64)
        exact = want.astype(np.float16).astype(np.float64)
        assert np.all(np.abs(got64 - want) <= 0.5 * _ulp16(want) * (1 + 2e-3))
        assert np.mean(got64 == exact) > 0.998
    # before the rounding the binary32 sequences are good to a few units in the last place
    np.testing.assert_allclose(npo.radius_f32(np.arange(n)), want_r, rtol=4e-7)
    c32, s32 = npo.cos_sin_f32(np.arange(n))
    np.testing.assert_allclose(c32, np.cos(theta), rtol=3e-7)
    np.testing.assert_allclose(s32, np.sin(theta), rtol=3e-7)
    # extremes and symmetry: largest radius sqrt(2 * 15 ln 2) = 4.56; inside the first quadrant the mirror
    # image about pi/4; a quarter turn maps (c, s) to (-s, c); the signs of the four quadrants
    assert float(R[0]) == float(np.float16(np.sqrt(30 * np.log(2.0)))) and R[-1] > 0
    assert np.all(np.diff(R.astype(np.float64)) <= 0)
    q = n // 4
    assert np.array_equal(C[:q], S[:q][::-1])
    assert np.array_equal(C[q:], -S[:-q]) and np.array_equal(S[q:], C[:-q])
    for k, (cs, ss) in enumerate(((1, 1), (-1, 1), (-1, -1), (1, -1))):
        assert np.all(np.sign(C[k * q:(k + 1) * q]) == cs) and np.all(np.sign(S[k * q:(k + 1) * q]) == ss)
    assert np.all(C != 0) and np.all(S != 0)
    # the C oracle holds the same tables
    for i in list(range(0, n, 509)) + [0, 1, n - 1]:
        assert c_oracle.radius_half(i) == int(R[i].view(np.uint16))
    for i in list(range(0, n, 127)) + [0, 2047, 2048, 4095, 4096, 8191, 8192, 12_287, 12_288, n - 1]:
        assert c_oracle.cos_half(i) == int(C[i].view(np.uint16))
        assert c_oracle.sin_half(i) == int(S[i].view(np.uint16))


def test_normal_entry_is_box_muller_in_fp16(c_oracle):
    # entry = fp16(R[x] * C[a] or S[a]); against Box-Muller in float64 with the same uniform
    # u = (x + 1/2) / 2^14 and the same angle: each factor is off by at most 2^-11 of itself (half
    # an fp16 step), the rounding of the product adds half a step
    rng = np.random.default_rng(7)
    w = rng.integers(0, 2**32, size=20_000, dtype=np.uint64).astype(np.uint32)
    w[:6] = [0, 0xFFFFFFFF, 0x7FFE0000, 0x0000FFFC, 0x80010003, 0x7FFEFFFC]
    x = ((w >> 17) & 0x3FFF).astype(np.float64)
    a = ((w >> 2) & 0x3FFF).astype(np.float64)
    r = np.sqrt(-2.0 * np.log((x + 0.5) / 2.0**14))
    theta = (a + 0.5) * (2 * np.pi) / 2.0**14
    R, C, S = npo.normal_tables()
    for sine, trig, tab in ((False, np.cos(theta), C), (True, np.sin(theta), S)):
        z = npo.normal_from_word(w, np.full(w.shape, sine))
        assert z.dtype == np.float16
        want = r * trig
        err = np.abs(z.astype(np.float64) - want)
        assert np.all(err <= (2.0**-10 * np.abs(want) + 0.5 * _ulp16(want)) * (1 + 1e-3))
        assert np.median(err / _ulp16(want)) < 0.5
        # bits 0, 1, 16 and 31 of the word are not part of any field
        assert np.array_equal(z, npo.normal_from_word(w ^ np.uint32(0x80010003), np.full(w.shape, sine)))
        # the definition itself, restated with exact rational arithmetic on a sample
        from fractions import Fraction
        for i in range(0, 20_000, 401):
            p = Fraction(float(R[int(x[i])])) * Fraction(float(tab[int(a[i])]))
            lo = np.float16(float(p))  # float(p) is exact (22 significant bits)
            assert float(z[i]) == float(lo)
            assert c_oracle.normal_from_word(int(w[i]), sine) == float(z[i])
            assert c_oracle.normal_from_word(int(w[i]) ^ 0x80010003, sine) == float(z[i])


def test_normal_block_uses_every_word_for_one_pair(c_oracle):
    # one tile of 8 features = one Philox block: entries (2i, 2i + 1) come from word i
    seed, col = 5, 9
    words = c_oracle.philox([0, c_oracle.stream_name(seed, col, 0), 0, 0], [seed, 0])
    colv = c_oracle.materialize(seed, 1, 8, 0, 8, col, 1, G)[:, 0]
    for e in range(8):
        assert colv[e] == c_oracle.normal_from_word(words[e // 2], e % 2)
    # and the second block of the stream serves features 8..15
    words1 = c_oracle.philox([1, c_oracle.stream_name(seed, col, 0), 0, 0], [seed, 0])
    colv = c_oracle.materialize(seed, 1, 16, 8, 8, col, 1, G)[:, 0]
    for e in range(8):
        assert colv[e] == c_oracle.normal_from_word(words1[e // 2], e % 2)


def test_half_rounding_matches_numpy_float16(c_oracle):
    rng = np.random.default_rng(9)
    vals = np.concatenate(
        [
            rng.standard_normal(3000).astype(np.float32) * 2,
            rng.standard_normal(500).astype(np.float32) * 1e-4,   # fp16 subnormals
            np.array([0.0, -0.0, 1.0, -1.0, 5.77, 6.1e-5, 5.96e-8, 2.98e-8, 2.99e-8, 1.00048828125], np.float32),
        ]
    )
    for v in vals:
        assert c_oracle.half_bits(float(v)) == int(np.float32(v).astype(np.float16).view(np.uint16))


def test_normal_entries_are_fp16_standard_normals(c_oracle):
    S = c_oracle.materialize(3, 256, 1 << 20, 0, 8192, 0, 32, G).astype(np.float64)
    assert np.array_equal(S.astype(np.float16).astype(np.float64), S)   # exactly fp16 values
    n = S.size
    assert abs(S.mean()) < 5 / math.sqrt(n)
    assert abs(S.var() - 1.0) < 5 * math.sqrt(2.0 / n) + 1e-6
    assert abs((S**4).mean() - 3.0) < 0.1
    from scipy import stats

    assert stats.kstest(S.ravel()[:50_000], "norm").pvalue > 1e-3
    # the cos and sin branches of one pair are uncorrelated, so are neighbouring columns
    assert abs(np.corrcoef(S[0::2].ravel(), S[1::2].ravel())[0, 1]) < 5 / math.sqrt(n / 2)
    # and their squares add up to the squared radius: chi-square with two degrees of freedom
    r2 = S[0::2].ravel() ** 2 + S[1::2].ravel() ** 2
    assert stats.kstest(r2[:50_000], "chi2", args=(2,)).pvalue > 1e-3
    # tails: the radius grid ends at sqrt(30 ln 2) = 4.56
    assert np.abs(S).max() <= 4.57 and np.abs(S).max() > 3.5
    assert abs(np.corrcoef(S[:, 0], S[:, 1])[0, 1]) < 5 / math.sqrt(S.shape[0])
