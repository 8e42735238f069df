"""Pins oracle/serialize.py without the reference: hand values, brute force on Python integers, and the properties
that define a Hilbert curve (bijection, face-adjacent steps, fixed end points)."""
import itertools

import numpy as np
import pytest

from oracle import serialize as oz


def cube(k):
    r = range(1 << k)
    return np.array([(0, x, y, z) for x, y, z in itertools.product(r, r, r)], dtype=np.int32)


def morton_bruteforce(b, x, y, z, bl):
    code = 0
    for i in range(bl):
        code |= ((x >> i) & 1) << (3 * i + 2) | ((y >> i) & 1) << (3 * i + 1) | ((z >> i) & 1) << (3 * i)
    return code | (b << (3 * bl))


def test_z_order_hand_values():
    c = np.array([(0, 1, 0, 0), (0, 0, 1, 0), (0, 0, 0, 1), (0, 3, 0, 0), (0, 0, 0, 3), (0, 7, 7, 7), (1, 0, 0, 0),
                  (2, 5, 2, 6)], dtype=np.int32)
    # x -> bit 2 of each triple, y -> bit 1, z -> bit 0; batch above 3*3 bits
    # (2, 5, 2, 6): x=101, y=010, z=110 -> triples (msb first) 101 011 100 = 0o534, batch 2 << 9
    want = [4, 2, 1, 0b100100, 0b001001, 511, 512, (2 << 9) | 0o534]
    assert oz.encode(c, 3, "z_order").tolist() == want


@pytest.mark.parametrize("bl", [1, 2, 5, 10, 11, 21])
def test_z_order_matches_bitwise_bruteforce(bl):
    rng = np.random.default_rng(bl)
    n = 500
    c = np.concatenate([rng.integers(0, 1 << min(2, 64 - 3 * bl), (n, 1)), rng.integers(0, 1 << bl, (n, 3))],
                       axis=1).astype(np.int32)
    got = oz.encode(c, bl, "z_order", np.int64).view(np.uint64)
    want = [morton_bruteforce(*[int(v) for v in row], bl) for row in c]
    assert got.tolist() == want
    assert np.array_equal(oz.decode(got.view(np.int64), bl, "z_order"), c)


def test_hilbert_first_order_octants_by_hand():
    # order 1: no "excess work" to undo; transpose = Gray encode: bits (x, x^y, x^y^z) -> index 4x + 2(x^y) + (x^y^z).
    # Solving index 0..7 for (x, y, z) gives the walk below (each step flips one coordinate).
    walk = [(0, 0, 0), (0, 0, 1), (0, 1, 1), (0, 1, 0), (1, 1, 0), (1, 1, 1), (1, 0, 1), (1, 0, 0)]
    c = np.array([(0,) + w for w in walk], dtype=np.int32)
    assert oz.encode(c, 1, "hilbert").tolist() == list(range(8))
    assert np.array_equal(oz.decode(np.arange(8, dtype=np.int64), 1, "hilbert"), c)


@pytest.mark.parametrize("k", [1, 2, 3, 4])
def test_hilbert_is_a_hilbert_curve(k):
    c = cube(k)
    code = oz.encode(c, k, "hilbert")
    n = 8 ** k
    assert sorted(code.tolist()) == list(range(n))                 # bijection onto 0 .. 8^k - 1
    walk = c[np.argsort(code)][:, 1:].astype(np.int64)
    steps = np.abs(np.diff(walk, axis=0))
    assert np.all(steps.sum(axis=1) == 1)                          # every step moves to a face neighbour
    assert walk[0].tolist() == [0, 0, 0]
    assert walk[-1].tolist() == [(1 << k) - 1, 0, 0]               # the two ends share an edge of the cube along x
    # self-similarity: each run of 8^(k-1) consecutive codes stays inside one octant, octants in first-order sequence
    if k > 1:
        octant = (walk >> (k - 1)).reshape(8, -1, 3)
        assert np.all(octant == octant[:, :1, :])
        first_order = oz.decode(np.arange(8, dtype=np.int64), 1, "hilbert")[:, 1:]
        assert np.array_equal(octant[:, 0, :], first_order)
    assert np.array_equal(oz.decode(code, k, "hilbert"), c)


@pytest.mark.parametrize("mode", oz.MODES)
@pytest.mark.parametrize("bl", [0, 1, 7, 10, 11, 16, 21])
def test_round_trip_with_batches(mode, bl):
    rng = np.random.default_rng(100 + bl)
    n = 2000
    batch_bits = min(3, 64 - 3 * bl)
    c = np.concatenate([rng.integers(0, 1 << batch_bits, (n, 1)),
                        rng.integers(0, 1 << bl, (n, 3)) if bl else np.zeros((n, 3), dtype=np.int64)],
                       axis=1).astype(np.int32)
    code = oz.encode(c, bl, mode, np.int64)
    assert np.array_equal(oz.decode(code, bl, mode), c)
    if batch_bits + 3 * bl <= 32:
        code32 = oz.encode(c, bl, mode, np.int32)
        assert code32.dtype == np.int32
        assert np.array_equal(code32.view(np.uint32).astype(np.uint64), code.view(np.uint64))
        assert np.array_equal(oz.decode(code32, bl, mode), c)


def test_hilbert_corner_cube_holds_the_first_codes():
    # The curve starts at the origin and fills one octant before the next, recursively: whatever the order, the corner
    # cube [0, 2^k)^3 holds exactly the first 8^k codes.
    k = 2
    c = cube(k)
    for order in (k, k + 1, k + 3):
        code = oz.encode(c, order, "hilbert")
        assert sorted(code.tolist()) == list(range(8 ** k))
        assert code[0] == 0


def test_code_width_rule():
    assert oz.code_dtype((1, 1, 1024, 1024, 1024)) == np.int32      # 30 bits
    assert oz.code_dtype((4, 1, 1024, 1024, 1024)) == np.int32      # 32 bits
    assert oz.code_dtype((5, 1, 1024, 1024, 1024)) == np.int64      # 33 bits
    assert oz.code_dtype((1, 1, 2048, 16, 16)) == np.int64
    assert oz.bit_lengths((1, 1, 1, 1, 1)) == (0, 0)
    with pytest.raises(ValueError):
        oz.code_dtype((2, 1, 1 << 22, 4, 4))


def test_reorder_coords_sorts_by_code():
    rng = np.random.default_rng(5)
    c = np.unique(np.concatenate([rng.integers(0, 2, (300, 1)), rng.integers(0, 16, (300, 3))], axis=1), axis=0).astype(np.int32)
    for mode in oz.MODES:
        r = oz.reorder_coords(c, 4, mode)
        code = oz.encode(r, 4, mode).astype(np.int64)
        assert np.all(np.diff(code) > 0)
        assert sorted(map(tuple, r.tolist())) == sorted(map(tuple, c.tolist()))
