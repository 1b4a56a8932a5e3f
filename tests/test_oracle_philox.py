"""Pins the Philox core, the stream-seed formula and the tiling of both oracles (and of the
library's host code) against published vectors and closed forms."""
import numpy as np
import pytest

from oracle import jl_oracle as npo

# Random123 v1.09 kat_vectors, lines "philox4x32 10 ...": counter, key -> output
KAT = [
    ([0, 0, 0, 0], [0, 0], [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]),
    ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
    (
        [0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344],
        [0xA4093822, 0x299F31D0],
        [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1],
    ),
]


@pytest.mark.parametrize("ctr,key,expect", KAT)
def test_philox_kat_c(c_oracle, ctr, key, expect):
    assert c_oracle.philox(ctr, key) == expect


@pytest.mark.parametrize("ctr,key,expect", KAT)
def test_philox_kat_numpy(ctr, key, expect):
    assert npo.philox4x32_10(ctr, key).tolist() == expect


def test_philox_c_vs_numpy_random(c_oracle):
    rng = np.random.default_rng(1)
    ctr = rng.integers(0, 2**32, size=(200, 4), dtype=np.uint64).astype(np.uint32)
    key = rng.integers(0, 2**32, size=(200, 2), dtype=np.uint64).astype(np.uint32)
    out = npo.philox4x32_10(ctr, key)
    for i in range(200):
        assert c_oracle.philox(ctr[i], key[i]) == out[i].tolist()


def test_philox_is_a_bijection_of_the_counter_low_word(c_oracle):
    # distinct counters under one key give distinct blocks (Philox is a permutation)
    key = np.tile(np.array([[123, 0]], dtype=np.uint32), (4096, 1))
    ctr = np.zeros((4096, 4), dtype=np.uint32)
    ctr[:, 0] = np.arange(4096)
    out = npo.philox4x32_10(ctr, key)
    assert len({tuple(r) for r in out.tolist()}) == 4096


def test_stream_name_closed_form(c_oracle):
    # fast_jl/random.cuh:15-17: seed + 658105236*column + 359124577*tile, uint32 wrap
    cases = [(0, 0, 0), (42, 1, 0), (42, 0, 1), (7, 4095, 255), (0xFFFFFFFF, 15359, 255), (10**8, 513, 107)]
    for seed, col, tile in cases:
        expect = (seed + 658105236 * col + 359124577 * tile) % 2**32
        assert c_oracle.stream_name(seed, col, tile) == expect
        assert int(npo.stream_name(seed, col, tile)) == expect
    # hand-computed: 42 + 658105236 = 658105278 ; 42 + 359124577 = 359124619
    assert c_oracle.stream_name(42, 1, 0) == 658105278
    assert c_oracle.stream_name(42, 0, 1) == 359124619
    # wrap: 658105236 * 7 = 4606736652 -> mod 2^32 = 311769356
    assert c_oracle.stream_name(0, 7, 0) == 311769356


def test_stream_block_is_philox_with_the_name_in_the_counter(c_oracle):
    # block n of the stream named s under a projector seed: counter (n, s, 0, 0), key (seed, 0)
    for seed, name, n in [(0, 0, 0), (42, 658105278, 3), (0xFFFFFFFF, 0x12345678, 0xFFFFFFFF)]:
        want = c_oracle.philox([n, name, 0, 0], [seed, 0])
        assert c_oracle.stream_block(seed, name, n) == want
        assert npo.stream_blocks(seed, name, n).tolist() == want
    # Random123's known-answer vector with zero counter and key, read as block 0 of stream 0 of
    # seed 0 (the other published vectors have counter and key words this entry point keeps zero)
    assert c_oracle.stream_block(0, 0, 0) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]


def test_tiling_matches_reference_iteration_counts(c_oracle):
    # fts = ceil(P / min(P, T)) (fast_jl/fast_jl.cu:42, fast_jl_kernel.cuh:124); the counts of
    # 256-feature iterations per tile for the benchmark shapes at T = 256
    for P, T, fts, iters in [
        (4_825_610, 256, 18_851, 74),
        (11_689_512, 256, 45_663, 179),
        (27_370_560, 256, 106_917, 418),
        (1_000, 256, 4, 1),
        (25, 256, 1, 1),
        (10_240, 108, 95, 1),
    ]:
        tiles, size = c_oracle.tiling(P, T)
        assert (tiles, size) == (min(P, T), fts)
        assert npo.tiling(P, T) == (min(P, T), fts)
        assert -(-size // 256) == iters
        assert tiles * size >= P
