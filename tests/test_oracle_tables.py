"""Pins the C restatement of the integer tables (oracle/subm_ref.c) against known answers,
independent definition-level builders and brute force.  CPU only."""
import numpy as np
import pytest

from flexgemm_amd.workloads import reference_test_shell, shell_coords
from oracle import definitions as df
from oracle import neighbor as nb

EMPTY = 0xFFFFFFFF


def _py_fmix32(k):
    k &= 0xFFFFFFFF
    k ^= k >> 16
    k = (k * 0x85EBCA6B) & 0xFFFFFFFF
    k ^= k >> 13
    k = (k * 0xC2B2AE35) & 0xFFFFFFFF
    k ^= k >> 16
    return k


def test_murmur3_finaliser_known_answers():
    # MurmurHash3 fmix32 / fmix64 known answers (public algorithm, values fixed by its constants)
    assert nb.fmix32(0) == 0
    assert nb.fmix32(1) == 0x514E28B7
    assert nb.fmix32(2) == 0x30F4C306
    assert nb.fmix64(0) == 0
    assert nb.fmix64(1) == 0xB456BCFC34C2CB2C
    # fmix32 is a bijection on 32-bit words: spot-check injectivity and agreement with a bignum restatement
    rng = np.random.default_rng(0)
    xs = rng.integers(0, 2 ** 32, size=2000, dtype=np.uint64)
    ys = {nb.fmix32(int(x)) for x in xs}
    assert len(ys) == len(set(int(x) for x in xs))
    for x in xs[:200]:
        assert nb.fmix32(int(x)) == _py_fmix32(int(x))


@pytest.mark.parametrize("key_bits", [32, 64])
def test_hash_round_trip(key_bits):
    # reference tests/hashmap.py:69 -- lookup(insert(k, v)) == v; absent / out-of-grid -> all ones
    res = 16
    coords = reference_test_shell(res, batch=2)
    rng = np.random.default_rng(1)
    coords = coords[rng.permutation(len(coords))]
    vals = rng.integers(0, 2 ** 31, size=len(coords)).astype(np.uint32)
    t = nb.HashTable(2 * len(coords), key_bits)
    t.insert_3d(coords, vals, res, res, res)
    assert (t.lookup_3d(coords, res, res, res) == vals).all()
    absent = np.array([[0, 0, 0, 0], [1, res // 2, res // 2, res // 2], [0, -1, 3, 3], [0, 3, 3, res]], dtype=np.int32)
    assert (t.lookup_3d(absent, res, res, res) == EMPTY).all()
    # load factor 1.0 still terminates and round-trips (linear probing with wrap-around)
    t = nb.HashTable(len(coords), key_bits)
    t.insert_3d(coords, vals, res, res, res)
    assert (t.lookup_3d(coords, res, res, res) == vals).all()


def test_key_width_rule():
    assert nb.key_bits_for((1, 8, 1024, 1024, 1024)) == 32
    assert nb.key_bits_for((4, 8, 1024, 1024, 1024)) == 64          # 2^32 is not < 2^32
    assert nb.key_bits_for((1, 8, 2048, 2048, 1023)) == 32


@pytest.mark.parametrize("res", [1, 2, 4, 8, 16, 32])
def test_neighbor_map_vs_definitions(res):
    # reference tests/submconv/neighbor_cache.py:63-93 sweeps this geometry
    coords = reference_test_shell(res)
    shape = (1, 0, res, res, res)
    got = nb.neighbor_map(coords, shape)
    assert got.dtype == np.uint32 and got.shape == (len(coords), 27)
    assert (got == df.neighbor_map_searchsorted(coords, shape)).all()
    if res <= 16:
        assert (got == df.neighbor_map_bruteforce(coords, shape)).all()
    # centre column is the voxel itself; symmetry map[n, v] = m <=> map[m, 26 - v] = n
    assert (got[:, 13] == np.arange(len(coords))).all()
    n_idx, v_idx = np.nonzero(got != EMPTY)
    assert (got[got[n_idx, v_idx], 26 - v_idx] == n_idx).all()


def test_neighbor_map_shuffled_batched_dilated_and_uint64():
    rng = np.random.default_rng(5)
    res = 12
    coords = reference_test_shell(res, batch=3)
    coords = coords[rng.permutation(len(coords))]
    for ks, dil in [((3, 3, 3), (1, 1, 1)), ((3, 3, 3), (2, 1, 3)), ((1, 3, 5), (1, 2, 1)), ((1, 1, 1), (1, 1, 1))]:
        shape = (3, 0, res, res, res)
        got = nb.neighbor_map(coords, shape, ks, dil)
        assert (got == df.neighbor_map_bruteforce(coords, shape, ks, dil)).all(), (ks, dil)
    # a grid so large that keys need 64 bits (B*W*H*D >= 2^32); voxels sit near the far corner
    big = (2, 0, 2048, 2048, 1024)
    far = coords.copy()
    far[:, 0] %= 2
    far[:, 1] += 2048 - res
    far[:, 2] += 2048 - res
    far[:, 3] += 1024 - res
    assert nb.key_bits_for(big) == 64
    _, uniq = np.unique(far, axis=0, return_index=True)
    far = far[np.sort(uniq)]
    assert (nb.neighbor_map(far, big) == df.neighbor_map_bruteforce(far, big)).all()


def test_neighbor_map_benchmark_shells_counts():
    # N and L of the benchmark geometry (res 64: 10 208 voxels, 105 488 valid pairs)
    coords = shell_coords(64)
    assert len(coords) == 10208
    m = nb.neighbor_map(coords, (1, 64, 64, 64, 64))
    assert int((m != EMPTY).sum()) == 105488
    assert (m == df.neighbor_map_searchsorted(coords, (1, 64, 64, 64, 64))).all()
    assert len(shell_coords(128)) == 42608


@pytest.mark.parametrize("res", [1, 2, 8, 32])
def test_codes_pairs_and_tile_masks(res):
    coords = reference_test_shell(res)
    rng = np.random.default_rng(res)
    coords = coords[rng.permutation(len(coords))]
    m = nb.neighbor_map(coords, (1, 0, res, res, res))
    gray, binary = nb.gray_binary(m)
    assert (gray == df.gray_code(m)).all()
    assert (binary == df.gray_to_binary(gray)).all()
    # Gray decode inverse: b ^ (b >> 1) == g
    b = binary.view(np.uint32)
    assert ((b ^ (b >> 1)) == gray.view(np.uint32)).all()
    assert ((gray >> 13) & 1).all()                     # centre bit always set for 3^3
    sig_i, sig_o, seg = nb.pair_lists(m)
    di, do, dseg = df.pair_lists(m)
    assert (sig_i == di).all() and (sig_o == do).all() and (seg == dseg).all()
    assert seg[0] == 0 and seg[-1] == (m != EMPTY).sum()
    s = nb.sorted_idx_canonical(binary)
    assert s.dtype == np.int64 and (np.sort(s) == np.arange(len(s))).all()
    assert (np.diff(binary[s]) >= 0).all()
    for blk in (2, 4, 32, 128, 256):
        vk, vseg = nb.tile_masks(gray, s, blk)
        dk, dsg = df.tile_masks(gray, s, blk)
        assert (vk == dk).all() and (vseg == dsg).all()
        # tie-order invariance: any permutation inside equal-code runs gives the same tables
        keys = binary[s].astype(np.int64) * (len(s) + 1) + rng.permutation(len(s))
        s2 = s[np.argsort(keys, kind="stable")]
        assert (np.diff(binary[s2]) >= 0).all()
        vk2, vseg2 = nb.tile_masks(gray, s2, blk)
        assert (vk2 == vk).all() and (vseg2 == vseg).all()


def test_empty_input():
    coords = np.zeros((0, 4), dtype=np.int32)
    m = df.neighbor_map_searchsorted(coords, (1, 0, 4, 4, 4))
    assert m.shape == (0, 27)
    sig_i, sig_o, seg = nb.pair_lists(m)
    assert len(sig_i) == 0 and (seg == 0).all()
