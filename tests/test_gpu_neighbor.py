"""GPU parity of the hash table, neighbor map and its post-processing against the CPU oracle (bit-exact)."""
import ctypes as C
import sys

import numpy as np
import pytest
import torch

import flex_gemm
from flex_gemm.ops.spconv import Algorithm, SubMConv3dFunction
from flexgemm_amd import _native as nat
from flexgemm_amd.ops.utils import init_hashmap
from flexgemm_amd.workloads import make_workload, reference_test_shell, shell_coords
from oracle import definitions as df
from oracle import neighbor as nb

pytestmark = pytest.mark.gpu
EMPTY = 0xFFFFFFFF


def _say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


@pytest.fixture(params=["hash", "sort"], autouse=True)
def neighbor_map_builder(request):
    """Every test of this file runs once per way of finding the neighbors: the tables must not depend on it."""
    flex_gemm.ops.spconv.set_neighbor_map_builder(request.param)
    yield request.param
    flex_gemm.ops.spconv.set_neighbor_map_builder("auto")


def _np(t):
    if t.dtype == torch.uint32:
        return t.cpu().view(torch.int32).numpy().view(np.uint32)
    return t.cpu().numpy()


def _check_cache(cache, coords_np, shape, needs_grad, blocks=(32, 128), ks=(3, 3, 3), dil=(1, 1, 1)):
    ref = nb.neighbor_cache(coords_np, tuple(shape), ks, dil, needs_grad=needs_grad, blocks=blocks)
    nmap = _np(cache.neighbor_map)
    assert cache.neighbor_map.dtype == torch.uint32
    assert np.array_equal(nmap, ref["neighbor_map"])
    assert cache.gray_code.dtype == torch.int32 and np.array_equal(_np(cache.gray_code), ref["gray_code"])
    s = _np(cache.sorted_idx)
    assert cache.sorted_idx.dtype == torch.int64
    assert np.array_equal(s, ref["sorted_idx"])          # stable order = canonical representative
    if needs_grad:
        assert np.array_equal(_np(cache.valid_signal_seg), ref["valid_signal_seg"])
        assert np.array_equal(_np(cache.valid_signal_i), ref["valid_signal_i"])
        assert np.array_equal(_np(cache.valid_signal_o), ref["valid_signal_o"])
    else:
        assert not hasattr(cache, "valid_signal_i")
    for b in blocks:
        assert np.array_equal(_np(cache.valid_kernel_callback(b)), ref[f"valid_kernel_{b}"])
        assert np.array_equal(_np(cache.valid_kernel_seg_callback(b)), ref[f"valid_kernel_seg_{b}"])


@pytest.mark.parametrize("res", [1, 2, 4, 8, 16, 32, 64])
@pytest.mark.parametrize("needs_grad", [False, True])
def test_cache_matches_oracle_reference_geometry(gpu_device, res, needs_grad):
    # the reference's own sweep: tests/submconv/neighbor_cache.py:63-93
    _say(f"neighbor cache res={res} needs_grad={needs_grad}")
    coords_np = reference_test_shell(res)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([1, 0, res, res, res])
    try:
        for algo in (Algorithm.MASKED_IMPLICIT_GEMM_SPLITK, Algorithm.MASKED_IMPLICIT_GEMM):
            flex_gemm.ops.spconv.set_algorithm(algo)
            cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), needs_grad)
            _check_cache(cache, coords_np, shape, needs_grad)
        # the other algorithms keep the neighbor map alone (reference submanifold_conv3d.py:59-71)
        for algo in (Algorithm.IMPLICIT_GEMM, Algorithm.IMPLICIT_GEMM_SPLITK, Algorithm.EXPLICIT_GEMM):
            flex_gemm.ops.spconv.set_algorithm(algo)
            cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), needs_grad)
            assert [k for k in vars(cache) if not k.startswith("_")] == ["neighbor_map"]
            assert np.array_equal(_np(cache.neighbor_map), nb.neighbor_map(coords_np, tuple(shape)))
        torch_cache = SubMConv3dFunction._compute_neighbor_cache_torch(coords, shape, (3, 3, 3), (1, 1, 1))
        assert torch.equal(cache.neighbor_map.view(torch.int32), torch_cache.neighbor_map.view(torch.int32))
    finally:
        flex_gemm.ops.spconv.set_algorithm(Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)


@pytest.mark.parametrize("res", [128, 256, 512])
def test_cache_matches_oracle_reference_geometry_large(gpu_device, res):
    # the upper part of the reference's sweep (tests/submconv/neighbor_cache.py:54 runs its shell up to res 512)
    _say(f"neighbor cache reference shell res={res}")
    coords_np = reference_test_shell(res)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([1, 0, res, res, res])
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    _check_cache(cache, coords_np, shape, True, blocks=(128,))


def test_repeated_voxels_give_the_same_map_with_both_builders(gpu_device, neighbor_map_builder):
    """A coordinate list that names some voxels twice: which of the equal rows a neighbor entry names is not fixed
    (the reference's hash insert lets the last writer win), but every entry must name a row with the right
    coordinates, exist exactly when such a row exists, and the middle entry must be the row itself."""
    rng = np.random.default_rng(5)
    res = 24
    base = reference_test_shell(res)
    coords_np = np.concatenate([base, base[rng.choice(len(base), 300, replace=False)], base[:7], base[:7]])
    coords_np = coords_np[rng.permutation(len(coords_np))]
    _say(f"neighbor map with repeated voxels, n={len(coords_np)} builder={neighbor_map_builder}")
    shape = torch.Size([1, 0, res, res, res])
    cache = SubMConv3dFunction._compute_neighbor_cache(torch.from_numpy(coords_np).to(gpu_device), shape, (3, 3, 3), (1, 1, 1), False)
    nmap = _np(cache.neighbor_map)
    n = len(coords_np)
    assert np.array_equal(nmap[:, 13], np.arange(n, dtype=np.uint32))
    present = {tuple(c) for c in coords_np.tolist()}
    offs = np.array([(0, dx, dy, dz) for dx in (-1, 0, 1) for dy in (-1, 0, 1) for dz in (-1, 0, 1)], dtype=np.int32)
    for v in range(27):
        want = coords_np + offs[v]
        found = nmap[:, v] != EMPTY
        assert np.array_equal(found, np.array([tuple(c) in present for c in want.tolist()]))
        assert np.array_equal(coords_np[nmap[found, v]], want[found])


def test_cache_shuffled_batched_dilated(gpu_device):
    rng = np.random.default_rng(7)
    res = 20
    coords_np = reference_test_shell(res, batch=3)
    coords_np = coords_np[rng.permutation(len(coords_np))]
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([3, 0, res, res, res])
    for ks, dil in [((3, 3, 3), (1, 1, 1)), ((3, 3, 3), (2, 1, 3)), ((1, 3, 5), (1, 2, 1)), ((1, 1, 1), (1, 1, 1)), ((3, 3, 1), (1, 1, 1))]:
        _say(f"neighbor cache ks={ks} dil={dil}")
        cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, ks, dil, True)
        _check_cache(cache, coords_np, shape, True, blocks=(2, 64, 100), ks=ks, dil=dil)


def test_grids_with_unequal_sides_and_steps_that_leave_the_grid(gpu_device, neighbor_map_builder):
    """Grids whose three sides differ (one of them 1 or 2 cells), every cell of the boundary occupied, and dilations whose
    steps reach past the far side or below zero from every voxel: a neighbor outside the grid is absent, never the voxel
    that the flattened key of the step would alias (x + 1 past the last column is not the first cell of the next row)."""
    rng = np.random.default_rng(11)
    for (w, h, d), batch in [((40, 6, 17), 2), ((1, 33, 9), 1), ((2, 2, 64), 3), ((7, 1, 1), 4), ((31, 32, 33), 1)]:
        cells = np.stack(np.meshgrid(np.arange(batch), np.arange(w), np.arange(h), np.arange(d), indexing="ij"), -1).reshape(-1, 4)
        keep = rng.random(len(cells)) < 0.6
        face = ((cells[:, 1] == 0) | (cells[:, 1] == w - 1) | (cells[:, 2] == 0) | (cells[:, 2] == h - 1) | (cells[:, 3] == 0)
                | (cells[:, 3] == d - 1))
        coords_np = np.ascontiguousarray(cells[keep | face][rng.permutation(int((keep | face).sum()))].astype(np.int32))
        coords = torch.from_numpy(coords_np).to(gpu_device)
        shape = torch.Size([batch, 0, w, h, d])
        for ks, dil in [((3, 3, 3), (1, 1, 1)), ((3, 3, 3), (w, h, d)), ((3, 3, 3), (max(w - 1, 1), max(h - 1, 1), max(d - 1, 1))),
                        ((5, 3, 1), (3, 5, 1)), ((1, 1, 9), (1, 1, 7)), ((3, 3, 3), (100, 1, 1000))]:
            _say(f"neighbor cache grid={(w, h, d)} batch={batch} ks={ks} dil={dil} builder={neighbor_map_builder}")
            cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, ks, dil, True)
            _check_cache(cache, coords_np, shape, True, blocks=(64,), ks=ks, dil=dil)


def test_large_kernel_explicit_and_uint64_keys(gpu_device):
    rng = np.random.default_rng(11)
    res = 12
    coords_np = reference_test_shell(res, batch=2)
    coords_np = coords_np[rng.permutation(len(coords_np))]
    # kernel volume 125 > 32: only the explicit algorithm accepts it
    flex_gemm.ops.spconv.set_algorithm(Algorithm.EXPLICIT_GEMM)
    try:
        _say("5x5x5 kernel, explicit")
        coords = torch.from_numpy(coords_np).to(gpu_device)
        shape = torch.Size([2, 0, res, res, res])
        cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (5, 5, 5), (1, 1, 1), False)
        assert np.array_equal(_np(cache.neighbor_map), df.neighbor_map_bruteforce(coords_np, tuple(shape), (5, 5, 5)))
    finally:
        flex_gemm.ops.spconv.set_algorithm(Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)
    with pytest.raises(AssertionError):
        SubMConv3dFunction._compute_neighbor_cache(coords, shape, (5, 5, 5), (1, 1, 1), False)
    # 64-bit keys: B*W*H*D >= 2^32
    _say("uint64 keys")
    big = torch.Size([2, 0, 2048, 2048, 1024])
    far = coords_np.copy()
    far[:, 1] += 2048 - res
    far[:, 2] += 2048 - res
    far[:, 3] += 1024 - res
    cache = SubMConv3dFunction._compute_neighbor_cache(torch.from_numpy(far).to(gpu_device), big, (3, 3, 3), (1, 1, 1), True)
    _check_cache(cache, far, big, True)


def test_empty_and_single_voxel(gpu_device):
    _say("empty input")
    coords = torch.zeros((0, 4), dtype=torch.int32, device=gpu_device)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, torch.Size([1, 0, 4, 4, 4]), (3, 3, 3), (1, 1, 1), True)
    assert cache.neighbor_map.shape == (0, 27) and cache.sorted_idx.shape == (0,)
    assert cache.valid_signal_i.shape == (0,) and _np(cache.valid_signal_seg).tolist() == [0] * 28
    assert cache.valid_kernel_callback(128).shape == (0,) and _np(cache.valid_kernel_seg_callback(128)).tolist() == [0]
    _say("single voxel")
    coords = torch.tensor([[0, 0, 0, 0]], dtype=torch.int32, device=gpu_device)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, torch.Size([1, 0, 1, 1, 1]), (3, 3, 3), (1, 1, 1), True)
    expect = np.full((1, 27), EMPTY, dtype=np.uint32)
    expect[0, 13] = 0
    assert np.array_equal(_np(cache.neighbor_map), expect)
    assert _np(cache.gray_code).tolist() == [1 << 13]
    assert _np(cache.valid_kernel_callback(128)).tolist() == [13]


@pytest.mark.parametrize("name,res", [("cfg2", 256), ("cfg4", 256), ("cfg3", 512)])
def test_cache_benchmark_shells(gpu_device, name, res):
    _say(f"neighbor cache {name} at res {res}")
    wl = make_workload(name, res=res, with_values=False)
    coords = wl.coords.to(gpu_device)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, wl.shape, (3, 3, 3), (1, 1, 1), True)
    _check_cache(cache, wl.coords.numpy(), wl.shape, True, blocks=(128,))


def test_full_size_res1024_properties(gpu_device):
    """Configuration 4 at full size (2.67 M shuffled voxels): exact equality with the oracle's map plus
    size-independent invariants of the derived tables."""
    _say("neighbor cache cfg4 res 1024")
    wl = make_workload("cfg4", with_values=False)
    assert wl.n == 2667120
    coords = wl.coords.to(gpu_device)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, wl.shape, (3, 3, 3), (1, 1, 1), True)
    nmap = _np(cache.neighbor_map)
    assert np.array_equal(nmap, nb.neighbor_map(wl.coords.numpy(), tuple(wl.shape)))
    n = wl.n
    L = int((nmap != EMPTY).sum())
    assert L == 28132992
    # symmetry: map[n, v] = m <=> map[m, 26 - v] = n
    rows, vs = np.nonzero(nmap != EMPTY)
    assert np.array_equal(nmap[nmap[rows, vs], 26 - vs], rows.astype(np.uint32))
    gray = _np(cache.gray_code)
    s = _np(cache.sorted_idx)
    assert np.array_equal(np.sort(s), np.arange(n))
    binary = df.gray_to_binary(gray)
    assert (np.diff(binary[s].astype(np.int64)) >= 0).all()
    seg = _np(cache.valid_signal_seg)
    assert seg[0] == 0 and seg[-1] == L and cache.valid_signal_i.shape[0] == L
    so, si = _np(cache.valid_signal_o), _np(cache.valid_signal_i)
    for v in (0, 13, 26):
        a, b = int(seg[v]), int(seg[v + 1])
        assert (np.diff(so[a:b].astype(np.int64)) > 0).all()
        assert np.array_equal(nmap[so[a:b], v], si[a:b])


@pytest.mark.parametrize("kbits,vbits", [(32, 32), (32, 64), (64, 32), (64, 64)])
def test_standalone_hash_round_trip(gpu_device, kbits, vbits):
    # reference tests/hashmap.py:9-69 -- insert random values, look them up again
    _say(f"hash round trip K={kbits} V={vbits}")
    L = nat.lib()
    kdt = torch.uint32 if kbits == 32 else torch.uint64
    vdt = torch.int32 if vbits == 32 else torch.int64
    for res in (1, 2, 16, 64):
        coords_np = reference_test_shell(res)
        m = len(coords_np)
        coords = torch.from_numpy(coords_np).to(gpu_device)
        table = 2 * m
        keys = torch.empty((table,), dtype=kdt, device=gpu_device)
        vals = torch.empty((table,), dtype=vdt, device=gpu_device)
        values = torch.randint(0, 2 ** 31 - 1, (m,), device=gpu_device).to(vdt)
        out = torch.empty_like(values)
        st = nat.stream()
        nat.check(L.fgx_hash_init(nat.ptr(keys), kbits, nat.sz(table), st))
        nat.check(L.fgx_hash_insert_3d(nat.ptr(keys), kbits, nat.ptr(vals), vbits, nat.sz(table), nat.ptr(coords),
                                       nat.ptr(values), nat.sz(m), res, res, res, st))
        nat.check(L.fgx_hash_lookup_3d(nat.ptr(keys), kbits, nat.ptr(vals), vbits, nat.sz(table), nat.ptr(coords),
                                       nat.ptr(out), nat.sz(m), res, res, res, st))
        assert torch.equal(out, values)
        # absent and out-of-grid queries give all ones
        q = torch.tensor([[0, -1, 0, 0], [0, 0, 0, res], [5, 0, 0, 0]], dtype=torch.int32, device=gpu_device)
        o = torch.zeros((3,), dtype=vdt, device=gpu_device)
        nat.check(L.fgx_hash_lookup_3d(nat.ptr(keys), kbits, nat.ptr(vals), vbits, nat.sz(table), nat.ptr(q),
                                       nat.ptr(o), nat.sz(3), res, res, res, st))
        assert (o == -1).all()
        # generic insert / lookup on pre-serialised keys, slot-for-slot identical to the CPU restatement's table
        flat = ((coords[:, 0].long() * res + coords[:, 1]) * res + coords[:, 2]) * res + coords[:, 3]
        k_in = flat.to(torch.int32).view(kdt) if kbits == 32 else flat.view(kdt)
        nat.check(L.fgx_hash_init(nat.ptr(keys), kbits, nat.sz(table), st))
        nat.check(L.fgx_hash_insert(nat.ptr(keys), kbits, nat.ptr(vals), vbits, nat.sz(table), nat.ptr(k_in),
                                    nat.ptr(values), nat.sz(m), st))
        o2 = torch.empty_like(values)
        nat.check(L.fgx_hash_lookup(nat.ptr(keys), kbits, nat.ptr(vals), vbits, nat.sz(table), nat.ptr(k_in),
                                    nat.ptr(o2), nat.sz(m), st))
        assert torch.equal(o2, values)
        if vbits == 32:
            # the SET of occupied slots with their keys is race-independent only per key's probe chain start;
            # what is fixed is that every key sits in its chain: check through the CPU restatement's lookup
            t = nb.HashTable(table, kbits)
            t.keys[:] = _np(keys.view(torch.int32) if kbits == 32 else keys.view(torch.int64)).view(t.keys.dtype)
            t.vals[:] = _np(vals).view(np.uint32)
            assert np.array_equal(t.lookup_3d(coords_np, res, res, res), _np(values).view(np.uint32))


def _morton_keys(coords_np):
    def spread(x):
        v = x.astype(np.uint64) & np.uint64(0xFFFF)
        v = (v | (v << np.uint64(16))) & np.uint64(0x0000FF0000FF)
        v = (v | (v << np.uint64(8))) & np.uint64(0x00F00F00F00F)
        v = (v | (v << np.uint64(4))) & np.uint64(0x0C30C30C30C3)
        v = (v | (v << np.uint64(2))) & np.uint64(0x249249249249)
        return v
    c = coords_np.astype(np.int64)
    return (c[:, 0].astype(np.uint64) << np.uint64(48)) | (spread(c[:, 1]) << np.uint64(2)) | (spread(c[:, 2]) << np.uint64(1)) | spread(c[:, 3])


@pytest.mark.parametrize("res,batch,shuffle", [(8, 1, False), (48, 2, True), (128, 1, True)])
def test_private_tile_order(gpu_device, res, batch, shuffle):
    """The kernels' private row order: Z-order ranks cut into chunks, stable mask sort inside each chunk."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    _say(f"private tile order res={res} batch={batch} shuffle={shuffle}")
    coords_np = shell_coords(res, batch=batch)
    if shuffle:
        coords_np = coords_np[np.random.default_rng(res).permutation(len(coords_np))]
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([batch, 0, res, res, res])
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), False)
    assert not hasattr(cache, "_tile_order")      # built on first use by a short-row layer
    cache._ensure_tile_order()
    order = _np(cache._tile_order)
    n = len(coords_np)
    assert order.dtype == np.int64 and np.array_equal(np.sort(order), np.arange(n))
    binary = df.gray_to_binary(_np(cache.gray_code)).astype(np.int64)
    rank_order = np.argsort(_morton_keys(coords_np), kind="stable")          # position -> voxel
    chunk = impl.LOCALITY_CHUNK_ROWS
    key = (np.arange(n) // chunk).astype(np.int64) << 32 | binary[rank_order]
    expect = rank_order[np.argsort(key, kind="stable")]
    assert np.array_equal(order, expect)
    # the public order is untouched and the public tile tables still describe it
    assert np.array_equal(_np(cache.sorted_idx), np.argsort(binary, kind="stable"))
    vk, seg = nb.tile_masks(_np(cache.gray_code), _np(cache.sorted_idx), 128)
    assert np.array_equal(_np(cache.valid_kernel_callback(128)), vk)
    assert np.array_equal(_np(cache.valid_kernel_seg_callback(128)), seg)


def test_cache_built_by_one_call_equals_the_cache_built_step_by_step(gpu_device):
    """fgx_subm_cache_build (map, codes, mask sort and pair lists enqueued by one call, the lists on the library's second
    stream from 393 216 voxels on) against the same cache made call by call: every public field equal, for training and
    inference caches, coordinates in scan order and shuffled, a dilated kernel, sizes on both sides of the second
    stream's threshold, and twice in a row (the second build reuses the first one's freed buffers)."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    rng = np.random.default_rng(3)
    cases = [("res 96 shuffled, training", reference_test_shell(96), 96, (3, 3, 3), (1, 1, 1), True, True),
             ("res 96, inference", reference_test_shell(96), 96, (3, 3, 3), (1, 1, 1), False, False),
             ("res 64 dilated 3 x 1 x 3", reference_test_shell(64), 64, (3, 1, 3), (2, 1, 2), True, True),
             ("res 448, training (two streams)", reference_test_shell(448), 448, (3, 3, 3), (1, 1, 1), True, False),
             ("res 448 shuffled, training (two streams)", reference_test_shell(448), 448, (3, 3, 3), (1, 1, 1), True, True)]
    old = (impl.CACHE_BUILD_ONE_CALL, flex_gemm.ops.spconv.NEIGHBOR_MAP_BUILDER if hasattr(flex_gemm.ops.spconv, "NEIGHBOR_MAP_BUILDER") else None)
    flex_gemm.ops.spconv.set_neighbor_map_builder("sort")
    try:
        for name, cn, res, ks, dil, grad, shuffle in cases:
            _say(f"cache by one call: {name} (n={len(cn)})")
            if shuffle:
                cn = cn[rng.permutation(len(cn))]
            coords = torch.from_numpy(np.ascontiguousarray(cn)).to(gpu_device)
            shape = torch.Size([1, 0, res, res, res])
            for rep in range(2):
                impl.CACHE_BUILD_ONE_CALL = False
                ref = SubMConv3dFunction._compute_neighbor_cache(coords, shape, ks, dil, grad)
                impl.CACHE_BUILD_ONE_CALL = True
                got = SubMConv3dFunction._compute_neighbor_cache(coords, shape, ks, dil, grad)
                fields = ["neighbor_map", "gray_code", "sorted_idx"] + (["valid_signal_seg", "valid_signal_i", "valid_signal_o"] if grad else [])
                for f in fields:
                    a, b = getattr(ref, f), getattr(got, f)
                    assert a.shape == b.shape and a.dtype == b.dtype, (name, f)
                    assert torch.equal(a.view(torch.int32) if a.dtype == torch.uint32 else a, b.view(torch.int32) if b.dtype == torch.uint32 else b), (name, f, rep)
                del ref, got
    finally:
        impl.CACHE_BUILD_ONE_CALL = old[0]
        flex_gemm.ops.spconv.set_neighbor_map_builder("auto")


def test_locality_order_over_the_grid_bits_equals_the_order_over_all_bits(gpu_device):
    """fgx_locality_order_grid sorts over the key bits a grid can differ in (on 32-bit keys when they fit): the same
    permutation as fgx_locality_order, which sorts over 16 bits per axis and 16 batch bits -- for a grid whose keys fit 32
    bits, one that needs 64, chunks of one rank (the curve's own order, also fgx_zorder_rows) and a handful of rows."""
    L = nat.lib()
    rng = np.random.default_rng(11)
    cases = [("32-bit keys", 3, 200, 9000, 8, 2, 512), ("64-bit keys", 5, 3000, 9000, 12, 3, 512),
             ("chunks of one rank", 2, 100, 5000, 7, 1, 1), ("five rows", 1, 64, 5, 6, 0, 8192)]
    for name, batch, res, n, bits, batch_bits, chunk in cases:
        _say(f"locality order over the grid's key bits: {name}")
        cn = np.concatenate([rng.integers(0, batch, (n, 1)), rng.integers(0, res, (n, 3))], axis=1).astype(np.int32)
        cn = np.unique(cn, axis=0)[rng.permutation(len(np.unique(cn, axis=0)))]
        n = len(cn)
        coords = torch.from_numpy(np.ascontiguousarray(cn)).to(gpu_device)
        binary = torch.from_numpy(rng.integers(0, 1 << 27, n).astype(np.int32)).to(gpu_device)
        with torch.cuda.device(gpu_device):
            ws = nat.workspace(L.fgx_locality_workspace_bytes(nat.sz(n)), gpu_device)
            wide = torch.empty((n,), dtype=torch.int64, device=gpu_device)
            tight = torch.empty_like(wide)
            nat.check(L.fgx_locality_order(nat.ptr(coords), nat.ptr(binary), nat.sz(n), C.c_int(27), C.c_int(chunk), nat.ptr(wide),
                                           nat.ptr(ws), nat.sz(ws.numel()), nat.stream()))
            nat.check(L.fgx_locality_order_grid(nat.ptr(coords), nat.ptr(binary), nat.sz(n), C.c_int(27), C.c_int(chunk),
                                                C.c_int(bits), C.c_int(batch_bits), nat.ptr(tight), nat.ptr(ws), nat.sz(ws.numel()),
                                                nat.stream()))
            assert torch.equal(wide, tight), name
            if chunk == 1:
                rows = torch.empty_like(wide)
                nat.check(L.fgx_zorder_rows(nat.ptr(coords), nat.sz(n), C.c_int(bits), C.c_int(batch_bits), nat.ptr(rows), nat.ptr(ws),
                                            nat.sz(ws.numel()), nat.stream()))
                assert torch.equal(wide, rows), name
        order = _np(wide)
        assert np.array_equal(np.sort(order), np.arange(n))
        rank_order = np.argsort(_morton_keys(cn), kind="stable")
        key = (np.arange(n) // chunk).astype(np.int64) << 32 | _np(binary).astype(np.int64)[rank_order]
        assert np.array_equal(order, rank_order[np.argsort(key, kind="stable")]), name


def test_sorted_builder_decides_the_key_sort_on_the_device(gpu_device, neighbor_map_builder):
    """fgx_subm_neighbor_map_sorted with presorted = 2 (what the cache builder passes) against presorted = 0 (always
    sort) and, where it applies, presorted = 1: coordinates in scan order, shuffled, in scan order but for the last two
    voxels, a single voxel, and more voxels than the device-side decision covers (it then sorts without asking)."""
    if neighbor_map_builder != "sort":
        pytest.skip("the sorted builder's own entry point")
    L = nat.lib()
    rng = np.random.default_rng(5)
    cases = []
    shell = reference_test_shell(96)
    cases.append(("scan order", shell, 96, True))
    cases.append(("shuffled", shell[rng.permutation(len(shell))], 96, False))
    swapped = shell.copy()
    swapped[[-1, -2]] = swapped[[-2, -1]]
    cases.append(("last two swapped", swapped, 96, False))
    cases.append(("one voxel", shell[:1].copy(), 96, True))
    big = shell_coords(1024)
    assert len(big) > (1 << 21)
    cases.append(("2.6 M voxels in scan order", big, 1024, True))
    for name, coords_np, res, ascending in cases:
        _say(f"sorted builder, key sort decided on the device: {name} (n={len(coords_np)})")
        coords = torch.from_numpy(np.ascontiguousarray(coords_np, dtype=np.int32)).to(gpu_device)
        n = coords.shape[0]
        maps = {}
        for mode in (0, 2) + ((1,) if ascending else ()):
            nmap = torch.full((n, 27), 0x7FFFFFFF, dtype=torch.int32, device=gpu_device)
            gray = torch.empty((n,), dtype=torch.int32, device=gpu_device)
            binary = torch.empty((n,), dtype=torch.int32, device=gpu_device)
            with torch.cuda.device(gpu_device):
                ws = nat.workspace(L.fgx_subm_neighbor_map_sorted_workspace_bytes(nat.sz(n), C.c_int(32), C.c_int(3), C.c_int(3)), gpu_device)
                ws.fill_(0xA5)          # stale flag words and tables must not matter
                nat.check(L.fgx_subm_neighbor_map_sorted(
                    nat.ptr(coords), nat.sz(n), C.c_int(1), C.c_int(res), C.c_int(res), C.c_int(res), C.c_int(3), C.c_int(3), C.c_int(3),
                    C.c_int(1), C.c_int(1), C.c_int(1), C.c_int(32), C.c_int(mode), nat.ptr(ws), nat.sz(ws.numel()),
                    nat.ptr(nmap), nat.ptr(gray), nat.ptr(binary), nat.stream()))
            torch.cuda.synchronize()
            maps[mode] = (nmap.cpu(), gray.cpu(), binary.cpu())
        for mode in maps:
            for got, want in zip(maps[mode], maps[0]):
                assert torch.equal(got, want), f"{name}: presorted={mode} differs from the always-sorting call"
        if n <= 200000:
            ref = nb.neighbor_cache(coords_np, (1, 8, res, res, res), (3, 3, 3), (1, 1, 1), needs_grad=False, blocks=())
            assert np.array_equal(maps[2][0].numpy().view(np.uint32), ref["neighbor_map"])
    with pytest.raises(ValueError):
        nat.check(L.fgx_subm_neighbor_map_sorted(
            nat.ptr(coords), nat.sz(n), C.c_int(1), C.c_int(res), C.c_int(res), C.c_int(res), C.c_int(3), C.c_int(3), C.c_int(3),
            C.c_int(1), C.c_int(1), C.c_int(1), C.c_int(32), C.c_int(3), nat.ptr(ws), nat.sz(ws.numel()),
            nat.ptr(nmap), nat.ptr(gray), nat.ptr(binary), nat.stream()))
