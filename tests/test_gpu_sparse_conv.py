"""GPU parity of the generic sparse convolution (stride / padding / dilation): output coordinates and both neighbor
maps bit-exact against the oracle's tables, forward / dgrad / wgrad / dbias against the explicit gather-GEMM oracle.

Tolerances as for the submanifold operator: max relative error <= 1e-2 for fp16 / bf16 and <= 1e-4 for fp32, against
the oracle evaluated in float64 on the same (already rounded) inputs.
"""
import contextlib
import math
import sys

import numpy as np
import pytest
import torch

import flex_gemm
from flex_gemm.ops.spconv import Algorithm, SparseConv3dFunction, sparse_conv3d
from flexgemm_amd.workloads import reference_test_shell
from oracle import explicit_gemm as eg
from oracle import neighbor as nb
from oracle import sparse_conv as sc

pytestmark = pytest.mark.gpu
TOL = {torch.float16: 1e-2, torch.bfloat16: 1e-2, torch.float32: 1e-4}

# (kernel, stride, padding, dilation): the reference's sweep (tests/spconv/neighbor_cache.py:80-86) and harder ones
GEOMS = [
    ((3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    ((3, 3, 3), (1, 1, 1), (2, 2, 2), (2, 2, 2)),
    ((2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1)),
    ((3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1)),
    ((3, 2, 1), (2, 1, 3), (1, 0, 2), (1, 2, 1)),
]


@pytest.fixture(params=["hash", "sort"], autouse=True)
def neighbor_map_builder(request):
    """Every test of this file runs once per way of finding the neighbors: nothing may depend on it."""
    flex_gemm.ops.spconv.set_neighbor_map_builder(request.param)
    yield request.param
    flex_gemm.ops.spconv.set_neighbor_map_builder("auto")


def _say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def _np(t):
    if t.dtype == torch.uint32:
        return t.cpu().view(torch.int32).numpy().view(np.uint32)
    return t.cpu().numpy()


@contextlib.contextmanager
def _algorithm(algo):
    flex_gemm.ops.spconv.set_algorithm(algo)
    try:
        yield
    finally:
        flex_gemm.ops.spconv.set_algorithm(Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)


def _force_schedule(wgrad=False, **fields):
    from flexgemm_amd import _native as nat

    @contextlib.contextmanager
    def cm():
        real = nat.table_lookup

        def forced(pass_kind, *a):
            s = real(pass_kind, *a)
            if (pass_kind == nat.PASS_WGRAD) == wgrad:
                for k, v in fields.items():
                    setattr(s, k, v)
            return s
        nat.table_lookup = forced
        try:
            yield
        finally:
            nat.table_lookup = real
    return cm()


def _assert_close(got, ref64, dtype, what):
    got = got.detach().cpu()
    tol = TOL[dtype]
    rms = max(float(ref64.double().pow(2).mean().sqrt()), 1e-30)
    e_metric = eg.calc_err(got.double() / rms, ref64.double() / rms)[0]
    e_scaled = eg.max_rel_err(got, ref64)
    assert e_metric <= tol and e_scaled <= tol, f"{what}: min(abs,rel)={e_metric:.3e} scaled={e_scaled:.3e} tol={tol}"


def _shell(res, batch=1, shuffle_seed=None):
    c = reference_test_shell(res, batch=batch) if batch > 1 else reference_test_shell(res)
    if shuffle_seed is not None:
        c = c[np.random.default_rng(shuffle_seed).permutation(len(c))]
    return np.ascontiguousarray(c)


@pytest.mark.parametrize("res", [1, 2, 4, 8, 16, 32, 64])
def test_output_coords_match_oracle(gpu_device, res):
    """The reference's own sweep (tests/spconv/out_coords.py:36-65, equality with the torch builder), plus the
    oracle's table and two batches in shuffled order."""
    for batch in (1, 2):
        coords_np = _shell(res, batch, shuffle_seed=res)
        shape = torch.Size([batch, 0, res, res, res])
        coords = torch.from_numpy(coords_np).to(gpu_device)
        for ks, st, pd, dl in GEOMS:
            _say(f"out coords res={res} batch={batch} K={ks} S={st} P={pd} D={dl}")
            got = SparseConv3dFunction._get_output_coords(coords, shape, ks, st, pd, dl)
            want = sc.output_coords(coords_np, tuple(shape), ks, st, pd, dl)
            assert got.dtype == torch.int32 and got.shape == want.shape
            assert np.array_equal(_np(got), want)
            host = SparseConv3dFunction._get_output_coords_torch(torch.from_numpy(coords_np), shape, ks, st, pd, dl)
            assert np.array_equal(host.numpy(), want)


def test_output_coords_wide_keys_and_empty(gpu_device):
    # an output grid of more than 2^32 cells needs 64-bit keys
    shape = torch.Size([3, 0, 2000, 2000, 2000])
    rng = np.random.default_rng(0)
    coords_np = np.unique(np.concatenate([rng.integers(0, 3, (500, 1)), rng.integers(0, 2000, (500, 3))], 1).astype(np.int32), axis=0)
    coords_np = coords_np[rng.permutation(len(coords_np))]
    coords = torch.from_numpy(np.ascontiguousarray(coords_np)).to(gpu_device)
    _say("out coords 64-bit keys")
    got = SparseConv3dFunction._get_output_coords(coords, shape, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1))
    assert np.array_equal(_np(got), sc.output_coords(coords_np, tuple(shape), (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)))
    _say("out coords, no input / no reachable cell")
    none = torch.empty((0, 4), dtype=torch.int32, device=gpu_device)
    assert SparseConv3dFunction._get_output_coords(none, shape, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)).shape == (0, 4)
    tiny = torch.zeros((1, 4), dtype=torch.int32, device=gpu_device)
    # kernel larger than the padded grid: the output grid is empty
    assert SparseConv3dFunction._get_output_coords(tiny, torch.Size([1, 0, 2, 2, 2]), (5, 5, 5), (1, 1, 1), (0, 0, 0), (1, 1, 1)).shape == (0, 4)


def _check_cache(cache, coords_np, oc_np, shape, geom, needs_grad, masked, sorted_bwd):
    ks, st, pd, dl = geom
    fwd, bwd = sc.neighbor_maps(coords_np, oc_np, tuple(shape), ks, st, pd, dl, with_bwd=needs_grad)
    assert cache.neighbor_map.dtype == torch.uint32 and np.array_equal(_np(cache.neighbor_map), fwd)
    if needs_grad:
        assert np.array_equal(_np(cache.neighbor_map_bwd), bwd)
    else:
        assert cache.neighbor_map_bwd is None
    if not masked:
        assert [k for k in vars(cache) if not k.startswith("_")] == ["neighbor_map", "neighbor_map_bwd"]
        return
    gray, binary = nb.gray_binary(fwd)
    assert np.array_equal(_np(cache.gray_code), gray)
    assert np.array_equal(_np(cache.sorted_idx), nb.sorted_idx_canonical(binary))
    if needs_grad:
        sig_i, sig_o, seg = nb.pair_lists(fwd)
        assert np.array_equal(_np(cache.valid_signal_seg), seg)
        assert np.array_equal(_np(cache.valid_signal_i), sig_i) and np.array_equal(_np(cache.valid_signal_o), sig_o)
    assert hasattr(cache, "sorted_idx_bwd") == (needs_grad and sorted_bwd)
    if needs_grad and sorted_bwd:
        gray_b, binary_b = nb.gray_binary(bwd)
        assert np.array_equal(_np(cache.gray_code_bwd), gray_b)
        assert np.array_equal(_np(cache.sorted_idx_bwd), nb.sorted_idx_canonical(binary_b))
        vk, seg = nb.tile_masks(gray_b, nb.sorted_idx_canonical(binary_b), 64)
        assert np.array_equal(_np(cache.valid_kernel_bwd_callback(64)), vk)
        assert np.array_equal(_np(cache.valid_kernel_bwd_seg_callback(64)), seg)
    vk, seg = nb.tile_masks(gray, nb.sorted_idx_canonical(binary), 128)
    assert np.array_equal(_np(cache.valid_kernel_callback(128)), vk)
    assert np.array_equal(_np(cache.valid_kernel_seg_callback(128)), seg)


@pytest.mark.parametrize("res", [1, 2, 4, 8, 16, 32])
@pytest.mark.parametrize("needs_grad", [False, True])
def test_neighbor_cache_matches_oracle(gpu_device, res, needs_grad):
    """Both maps and every derived table, for every algorithm value (reference: tests/spconv/neighbor_cache.py:77-121
    compares the forward map with the torch builder)."""
    coords_np = _shell(res, 2, shuffle_seed=7)
    shape = torch.Size([2, 0, res, res, res])
    coords = torch.from_numpy(coords_np).to(gpu_device)
    for geom in GEOMS:
        ks, st, pd, dl = geom
        oc_np = sc.output_coords(coords_np, tuple(shape), ks, st, pd, dl)
        oc = torch.from_numpy(oc_np).to(gpu_device)
        for algo in (Algorithm.MASKED_IMPLICIT_GEMM_SPLITK, Algorithm.IMPLICIT_GEMM, Algorithm.EXPLICIT_GEMM):
            _say(f"sparse cache res={res} grad={needs_grad} K={ks} S={st} P={pd} D={dl} {algo}")
            with _algorithm(algo):
                cache = SparseConv3dFunction._compute_neighbor_cache(coords, oc, shape, ks, st, pd, dl, needs_grad)
                _check_cache(cache, coords_np, oc_np, shape, geom, needs_grad, algo == Algorithm.MASKED_IMPLICIT_GEMM_SPLITK,
                             any(s != 1 for s in st))
        with _algorithm(Algorithm.EXPLICIT_GEMM):
            host = SparseConv3dFunction._compute_neighbor_cache_torch(torch.from_numpy(coords_np), torch.from_numpy(oc_np), shape,
                                                                     ks, st, pd, dl, needs_grad)
            _check_cache(host, coords_np, oc_np, shape, geom, needs_grad, False, False)


def _run_and_check(coords_np, shape, geom, ci, co, dtype, dev, seed, algo=Algorithm.MASKED_IMPLICIT_GEMM_SPLITK, out_coords_np=None,
                   use_bias=True):
    ks, st, pd, dl = geom
    g = torch.Generator().manual_seed(seed)
    m = len(coords_np)
    v = ks[0] * ks[1] * ks[2]
    given = out_coords_np is not None
    oc_np = out_coords_np if given else sc.output_coords(coords_np, tuple(shape), ks, st, pd, dl)
    feats = torch.randn(m, ci, generator=g).to(dtype)
    weight = (torch.randn(co, *ks, ci, generator=g) / math.sqrt(v * ci)).to(dtype)
    bias = torch.randn(co, generator=g).to(dtype)
    grad = torch.randn(len(oc_np), co, generator=g).to(dtype)
    fwd, bwd = sc.neighbor_maps(coords_np, oc_np, tuple(shape), ks, st, pd, dl)
    ref_out = sc.forward(feats.double(), fwd, weight.double(), bias.double() if use_bias else None)
    ref_gi, ref_gw, ref_gb = sc.backward(grad.double(), feats.double(), fwd, bwd, weight.double())
    with _algorithm(algo):
        f = feats.to(dev).requires_grad_(True)
        w = weight.to(dev).requires_grad_(True)
        b = bias.to(dev).requires_grad_(True) if use_bias else None
        coords = torch.from_numpy(coords_np).to(dev)
        oc_in = torch.from_numpy(oc_np).to(dev) if given else None
        out, oc, cache = sparse_conv3d(f, coords, shape, w, b, out_coords=oc_in, stride=st, padding=pd, dilation=dl)
        assert np.array_equal(_np(oc), oc_np)
        assert out.dtype == dtype and out.shape == (len(oc_np), co)
        out.backward(grad.to(dev))
        torch.cuda.synchronize()
        _assert_close(out, ref_out, dtype, "forward")
        _assert_close(f.grad, ref_gi, dtype, "dgrad")
        _assert_close(w.grad, ref_gw, dtype, "wgrad")
        assert f.grad.shape == feats.shape and w.grad.shape == weight.shape
        if use_bias:
            _assert_close(b.grad, ref_gb, dtype, "dbias")
        # the cache is reusable: same results from a second call that is handed the cache
        out2, _, _ = sparse_conv3d(f.detach(), coords, shape, w.detach(), None if b is None else b.detach(), neighbor_cache=cache,
                                   out_coords=oc_in, stride=st, padding=pd, dilation=dl)
        assert torch.equal(out2, out.detach())
    return cache


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("geom", GEOMS)
def test_conv_matches_oracle(gpu_device, dtype, geom):
    res = 20
    coords_np = _shell(res, 2, shuffle_seed=3)
    shape = torch.Size([2, 0, res, res, res])
    for ci, co in [(64, 64), (32, 128), (20, 12)]:
        _say(f"sparse conv geom={geom} ci={ci} co={co} {dtype}")
        _run_and_check(coords_np, shape, geom, ci, co, dtype, gpu_device, seed=ci + co)


def test_algorithm_values(gpu_device):
    res = 16
    coords_np = _shell(res, 1, shuffle_seed=5)
    shape = torch.Size([1, 0, res, res, res])
    for geom in (GEOMS[0], GEOMS[2]):
        for algo in (Algorithm.MASKED_IMPLICIT_GEMM_SPLITK, Algorithm.MASKED_IMPLICIT_GEMM, Algorithm.IMPLICIT_GEMM,
                     Algorithm.IMPLICIT_GEMM_SPLITK, Algorithm.EXPLICIT_GEMM):
            _say(f"sparse conv algorithm {algo} geom={geom}")
            _run_and_check(coords_np, shape, geom, 64, 64, torch.float16, gpu_device, seed=9, algo=algo,
                           use_bias=algo != Algorithm.IMPLICIT_GEMM)


def test_given_output_coords_and_unreached_rows(gpu_device):
    """Caller-chosen output cells: a shuffled half of the reachable ones plus cells no input reaches (their output is
    the bias, their gradient contribution nothing); inputs that reach no chosen output get a zero gradient."""
    res = 16
    coords_np = _shell(res, 1, shuffle_seed=2)
    shape = torch.Size([1, 0, res, res, res])
    geom = GEOMS[3]
    rng = np.random.default_rng(4)
    reach = sc.output_coords(coords_np, tuple(shape), *geom)
    wo, ho, do = sc.out_dims(tuple(shape), *geom)
    cells = np.stack(np.meshgrid(np.zeros(1, np.int32), np.arange(wo), np.arange(ho), np.arange(do), indexing="ij"), -1).reshape(-1, 4)
    unreached = np.asarray(sorted(set(map(tuple, cells)) - set(map(tuple, reach))), dtype=np.int32)[:17]
    given = np.concatenate([reach[rng.permutation(len(reach))[: len(reach) // 2]], unreached]).astype(np.int32)
    given = np.ascontiguousarray(given[rng.permutation(len(given))])
    for dtype in (torch.float16, torch.float32):
        _say(f"sparse conv given out_coords {dtype}")
        cache = _run_and_check(coords_np, shape, geom, 64, 32, dtype, gpu_device, seed=11, out_coords_np=given)
        assert hasattr(cache, "sorted_idx_bwd")


@pytest.mark.parametrize("geom", [GEOMS[0], GEOMS[2], GEOMS[3]])
def test_streaming_kernels_with_distinct_row_counts(gpu_device, geom):
    """The persistent streaming GEMM and wgrad kernels forced on maps whose rows and source rows differ in number."""
    res = 40
    coords_np = _shell(res, 1, shuffle_seed=8)
    shape = torch.Size([1, 0, res, res, res])
    _say(f"sparse conv streaming kernels geom={geom}")
    with _force_schedule(tile_rows=256, tile_cols=128, slab_bytes=128, splitk=1, stream=1), \
            _force_schedule(wgrad=True, tile_rows=128, tile_cols=128, block_rows=1024, stream=1):
        _run_and_check(coords_np, shape, geom, 128, 128, torch.float16, gpu_device, seed=13)


@pytest.mark.parametrize("geom", [GEOMS[0], GEOMS[2], GEOMS[3]])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_weight_gradient_sweep_with_distinct_row_counts(gpu_device, geom, dtype):
    """The wgrad sweep (a weight of one tile) forced on maps whose output rows and input rows differ in number, from
    shuffled coordinates: its plan only needs pair lists that ascend in the output row inside every offset."""
    res = 40
    coords_np = _shell(res, 1, shuffle_seed=8)
    shape = torch.Size([1, 0, res, res, res])
    for ci, co, tile, sub_rows in ((128, 128, 128, 256), (48, 64, 64, 2048)):
        _say(f"sparse conv wgrad sweep geom={geom} ci={ci} co={co} sub_rows={sub_rows} {dtype}")
        with _force_schedule(wgrad=True, tile_rows=tile, tile_cols=tile, block_rows=sub_rows, stream=2):
            _run_and_check(coords_np, shape, geom, ci, co, dtype, gpu_device, seed=17)


def test_empty_input(gpu_device):
    shape = torch.Size([1, 0, 8, 8, 8])
    none = torch.empty((0, 4), dtype=torch.int32, device=gpu_device)
    f = torch.empty((0, 16), dtype=torch.float16, device=gpu_device)
    w = torch.randn(8, 3, 3, 3, 16, dtype=torch.float16, device=gpu_device)
    _say("sparse conv, empty input")
    out, oc, cache = sparse_conv3d(f, none, shape, w, None, padding=(1, 1, 1))
    assert out.shape == (0, 8) and oc.shape == (0, 4) and cache.neighbor_map.shape == (0, 27)


@pytest.mark.parametrize("geom", [GEOMS[2], GEOMS[3]])
def test_strided_views_give_the_bits_of_their_dense_copies(gpu_device, geom):
    """Weight, bias and upstream gradient handed over as views with strides of their own."""
    ks, st, pd, dl = geom
    _say(f"sparse conv with strided arguments, geometry {geom}")
    dev = gpu_device
    res, ci, co = 24, 64, 40
    coords = torch.from_numpy(_shell(res)).to(dev)
    shape = torch.Size([1, ci, res, res, res])
    g = torch.Generator().manual_seed(5)
    f0 = torch.randn(coords.shape[0], ci, generator=g).half().to(dev)
    w0 = (torch.randn(co, *ks, ci, generator=g) / math.sqrt(ks[0] * ks[1] * ks[2] * ci)).half().to(dev)
    b0 = torch.randn(co, generator=g).half().to(dev)

    def step(w, b, make_grad):
        f = f0.clone().requires_grad_(True)
        out, oc, _ = sparse_conv3d(f, coords, shape, w, b, stride=st, padding=pd, dilation=dl)
        go = make_grad(out)
        out.backward(go)
        torch.cuda.synchronize()
        return out.detach(), f.grad, w.grad, b.grad, oc

    gen = torch.Generator(device=dev)
    dense = lambda out: torch.randn(out.shape, generator=gen.manual_seed(9), device=dev).to(out.dtype)
    ref = step(w0.clone().requires_grad_(True), b0.clone().requires_grad_(True), dense)
    ws = w0.permute(4, 1, 2, 3, 0).contiguous().permute(4, 1, 2, 3, 0).requires_grad_(True)
    bs = torch.stack([b0, b0], 1)[:, 0].requires_grad_(True)
    assert not ws.is_contiguous() and not bs.is_contiguous()
    got = step(ws, bs, lambda out: dense(out).t().contiguous().t())
    for name, a, r in zip(("output", "input gradient", "weight gradient", "bias gradient", "output coordinates"), got, ref):
        assert a.shape == r.shape and torch.equal(a, r), name


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("geom", [GEOMS[0], GEOMS[2], GEOMS[3]])
def test_relu_in_the_epilogue_equals_relu_after_the_operator(gpu_device, dtype, geom):
    """sparse_conv3d_relu against torch.relu(sparse_conv3d): same bits in the output and in every gradient."""
    from flex_gemm.ops.spconv import sparse_conv3d_relu
    res, ci, co = 24, 64, 96
    ks, st, pd, dl = geom
    coords_np = _shell(res, 2, shuffle_seed=7)
    shape = torch.Size([2, 0, res, res, res])
    g = torch.Generator().manual_seed(17)
    m = len(coords_np)
    v = ks[0] * ks[1] * ks[2]
    feats = torch.randn(m, ci, generator=g).to(dtype)
    weight = (torch.randn(co, *ks, ci, generator=g) / math.sqrt(v * ci)).to(dtype)
    bias = torch.randn(co, generator=g).to(dtype)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    results = []
    grad = None
    _say(f"fused relu, generic conv geom={geom} {dtype}")
    for fused in (False, True):
        f = feats.to(gpu_device).requires_grad_(True)
        w = weight.to(gpu_device).requires_grad_(True)
        b = bias.to(gpu_device).requires_grad_(True)
        if fused:
            out, oc, _ = sparse_conv3d_relu(f, coords, shape, w, b, stride=st, padding=pd, dilation=dl)
        else:
            out, oc, _ = sparse_conv3d(f, coords, shape, w, b, stride=st, padding=pd, dilation=dl)
            out = torch.relu(out)
        if grad is None:
            grad = torch.randn(out.shape, generator=g).to(dtype).to(gpu_device)
        out.backward(grad)
        torch.cuda.synchronize()
        results.append((out.detach(), f.grad, w.grad, b.grad, oc))
    for name, a, b_ in zip(("output", "dgrad", "wgrad", "dbias", "out_coords"), results[0], results[1]):
        assert torch.equal(a, b_), f"{name}: fused and composed results differ"
    assert (results[1][0] == 0).any() and (results[1][0] > 0).any()
