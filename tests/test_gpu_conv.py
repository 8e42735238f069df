"""GPU parity of the masked implicit GEMM (forward, dgrad, wgrad, dbias) against the explicit gather-GEMM oracle.

Tolerances (stated by the build's north star): max relative error <= 1e-2 for fp16 / bf16 and <= 1e-4 for fp32.
Two readings of "relative error" are asserted, both against the oracle evaluated in float64 on the same
(already rounded) inputs: max|d| / max|ref|, and the reference's own metric max(min(|d|, |d|/|ref|))
(tests/utils.py:28-32) applied to tensors divided by rms(ref) -- without that normalisation the metric's absolute
branch is a statement about the tensor's scale (weight gradients are sums over up to N rows), not about accuracy.
"""
import math
import sys

import numpy as np
import pytest
import torch

import flex_gemm
from flex_gemm.ops.spconv import Algorithm, SubMConv3dFunction, sparse_submanifold_conv3d
from flexgemm_amd.workloads import make_workload, reference_test_shell
from oracle import explicit_gemm as eg
from oracle import neighbor as nb

pytestmark = pytest.mark.gpu
TOL = {torch.float16: 1e-2, torch.bfloat16: 1e-2, torch.float32: 1e-4}


def _say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def _assert_close(got, ref64, dtype, what):
    got = got.detach().cpu()
    tol = TOL[dtype]
    rms = max(float(ref64.double().pow(2).mean().sqrt()), 1e-30)
    e_ref_metric = eg.calc_err(got.double() / rms, ref64.double() / rms)[0]
    e_scaled = eg.max_rel_err(got, ref64)
    assert e_ref_metric <= tol and e_scaled <= tol, f"{what}: min(abs,rel)={e_ref_metric:.3e} scaled={e_scaled:.3e} tol={tol}"
    return e_ref_metric, e_scaled


def _case(coords_np, ci, co, dtype, seed, ksize=(3, 3, 3), wscale=None):
    g = torch.Generator().manual_seed(seed)
    n = len(coords_np)
    v = ksize[0] * ksize[1] * ksize[2]
    feats = torch.randn(n, ci, generator=g).to(dtype)
    weight = (torch.randn(co, *ksize, ci, generator=g) * (wscale or 1.0 / math.sqrt(v * ci))).to(dtype)
    bias = torch.randn(co, generator=g).to(dtype)
    grad = torch.randn(n, co, generator=g).to(dtype)
    return feats, weight, bias, grad


def _run_and_check(coords_np, shape, ci, co, dtype, dev, seed=0, ksize=(3, 3, 3), dilation=(1, 1, 1), use_bias=True,
                   algo=Algorithm.MASKED_IMPLICIT_GEMM_SPLITK, cache=None):
    feats, weight, bias, grad = _case(coords_np, ci, co, dtype, seed, ksize)
    nmap = torch.from_numpy(nb.neighbor_map(coords_np, tuple(shape), ksize, dilation).view(np.int32))
    f64, w64, b64, g64 = feats.double(), weight.double(), bias.double(), grad.double()
    ref_out = eg.forward(f64, nmap, w64, b64 if use_bias else None)
    ref_gi, ref_gw, ref_gb = eg.backward(g64, f64, nmap, w64)
    flex_gemm.ops.spconv.set_algorithm(algo)
    try:
        f = feats.to(dev).requires_grad_(True)
        w = weight.to(dev).requires_grad_(True)
        b = bias.to(dev).requires_grad_(True) if use_bias else None
        coords = torch.from_numpy(coords_np).to(dev)
        out, cache = sparse_submanifold_conv3d(f, coords, shape, w, b, neighbor_cache=cache, dilation=dilation)
        assert out.dtype == dtype and out.shape == (len(coords_np), co)
        out.backward(grad.to(dev))
        torch.cuda.synchronize()
        errs = [_assert_close(out, ref_out, dtype, "forward"),
                _assert_close(f.grad, ref_gi, dtype, "dgrad"),
                _assert_close(w.grad, ref_gw, dtype, "wgrad")]
        assert w.grad.shape == weight.shape
        if use_bias:
            errs.append(_assert_close(b.grad, ref_gb, dtype, "dbias"))
    finally:
        flex_gemm.ops.spconv.set_algorithm(Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)
    return cache, errs


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("res,ci,co", [(16, 32, 32), (16, 64, 64), (32, 128, 128), (24, 64, 128), (24, 256, 32), (8, 1024, 64)])
def test_conv_matches_oracle(gpu_device, dtype, res, ci, co):
    _say(f"conv res={res} ci={ci} co={co} {dtype}")
    coords_np = reference_test_shell(res)
    _run_and_check(coords_np, torch.Size([1, ci, res, res, res]), ci, co, dtype, gpu_device, seed=res + ci)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("res,ci,co", [(32, 32, 32), (40, 24, 16), (48, 8, 32), (24, 32, 8), (20, 16, 24)])
def test_narrow_resident_gemm_matches_oracle(gpu_device, dtype, res, ci, co):
    """Forward and dgrad of narrow layers through the resident-row kernel (fgx_conv_narrow_gemm, forced on): rows of 16 to
    64 bytes on either side, a last chunk that is partly empty, against the float64 oracle; wgrad and dbias ride along on
    their usual kernels."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    _say(f"narrow resident res={res} ci={ci} co={co} {dtype}")
    coords_np = reference_test_shell(res)
    old = impl.spconv.NARROW_RESIDENT
    impl.spconv.NARROW_RESIDENT = "on"
    try:
        cache, _ = _run_and_check(coords_np, torch.Size([1, ci, res, res, res]), ci, co, dtype, gpu_device, seed=res + ci)
    finally:
        impl.spconv.NARROW_RESIDENT = old
    assert hasattr(cache, "_narrow_plan_buf"), "the resident-row kernel did not run"
    assert getattr(cache, "_narrow_overflows", None) == 0, "the weight gradient did not take the resident-row kernel"


@pytest.mark.parametrize("res,ksize,dilation", [(4, (3, 3, 3), (1, 1, 1)), (24, (3, 3, 1), (1, 1, 1)), (24, (1, 3, 3), (2, 1, 1)),
                                                (16, (1, 1, 1), (1, 1, 1))])
def test_narrow_resident_kernels_other_volumes_and_tiny_inputs(gpu_device, res, ksize, dilation):
    """The resident-row kernels with fewer voxels than one chunk, and with kernel volumes other than 27 (the offsets' loop
    is then not unrolled; the weight gradient's multipliers own eight offsets each, so nine offsets leave three of the
    four nearly idle, one offset three of them entirely)."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    _say(f"narrow resident res={res} ksize={ksize} dilation={dilation}")
    coords_np = reference_test_shell(res)
    old = impl.spconv.NARROW_RESIDENT
    impl.spconv.NARROW_RESIDENT = "on"
    try:
        cache, _ = _run_and_check(coords_np, torch.Size([1, 32, res, res, res]), 32, 16, torch.float16, gpu_device, seed=res,
                                  ksize=ksize, dilation=dilation)
    finally:
        impl.spconv.NARROW_RESIDENT = old
    assert hasattr(cache, "_narrow_plan_buf") and getattr(cache, "_narrow_overflows", None) == 0


def test_narrow_resident_wgrad_is_reproducible_and_falls_back_on_overflow(gpu_device):
    """fgx_conv_narrow_wgrad twice: same bits (fixed summation order); against the block-major kernel fp32 rounding of a
    different order.  A plan whose header counts overflowing chunks sends the weight gradient to the block-major kernel."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    _say("narrow resident wgrad reproducibility / fallback")
    res, ci, co = 40, 32, 24
    coords_np = reference_test_shell(res)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([1, ci, res, res, res])
    f, _, _, g = _case(coords_np, ci, co, torch.bfloat16, 59)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    fd, gd = f.to(gpu_device), g.to(gpu_device)
    old = impl.spconv.NARROW_RESIDENT
    try:
        impl.spconv.NARROW_RESIDENT = "on"
        a = impl._wgrad(gd, fd, cache, 27, with_bias=True, bias_offset=13)
        b = impl._wgrad(gd, fd, cache, 27, with_bias=True, bias_offset=13)
        assert cache["_narrow_overflows"] == 0
        impl.spconv.NARROW_RESIDENT = "off"
        c = impl._wgrad(gd, fd, cache, 27, with_bias=True, bias_offset=13)
        impl.spconv.NARROW_RESIDENT = "on"
        cache["_narrow_overflows"] = 3                # as if three chunks had overflowed
        d = impl._wgrad(gd, fd, cache, 27, with_bias=True, bias_offset=13)
    finally:
        impl.spconv.NARROW_RESIDENT = old
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    assert eg.max_rel_err(a[0].cpu(), c[0].cpu().double()) <= 1e-2 and eg.max_rel_err(a[1].cpu(), c[1].cpu().double()) <= 1e-2
    assert torch.equal(d[0], c[0]), "with overflowing chunks the block-major kernel runs"


def test_narrow_resident_gemm_relu_mask_and_overflowing_chunks(gpu_device):
    """The resident-row kernel with the fused ReLU and its bit mask; and with rows in a random order, where a chunk of 128
    rows has far more than 448 distinct sources, so that most sources are read from memory by the multipliers: the sums
    run over the same offsets in the same order, so the result is the same bit for bit as with the rows in Z-order."""
    import ctypes as C
    from flexgemm_amd import _native as nat
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    _say("narrow resident relu mask / overflow")
    res, c = 48, 32
    coords_np = reference_test_shell(res)
    n = coords_np.shape[0]
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([1, c, res, res, res])
    f, w, b, _ = _case(coords_np, c, c, torch.float16, 53)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), False)
    fd, wd, bd = f.to(gpu_device), w.to(gpu_device).reshape(c, 27, c), b.to(gpu_device)
    old = impl.spconv.NARROW_RESIDENT
    impl.spconv.NARROW_RESIDENT = "on"
    try:
        masks = []
        out = impl._gather_gemm(fd, wd, bd, cache, 0, False, activation=nat.ACT_RELU, relu_mask_out=masks)
    finally:
        impl.spconv.NARROW_RESIDENT = old
    assert hasattr(cache, "_narrow_plan_buf") and len(masks) == 1
    ref = torch.relu(eg.forward(f.double(), cache.neighbor_map.cpu().view(torch.int32), w.double(), b.double()))
    assert eg.max_rel_err(out.cpu(), ref) <= 1e-2
    bits = np.unpackbits(masks[0].cpu().numpy(), bitorder="little").reshape(n, c).astype(bool)
    assert np.array_equal(bits, (out.cpu().float() > 0).numpy()), "the mask is not 'output greater than zero'"
    # rows in a random order: chunks whose sources do not fit the slots
    L = nat.lib()
    order = torch.from_numpy(np.random.default_rng(5).permutation(n).astype(np.int64)).to(gpu_device)
    nmap = cache["neighbor_map"]
    plan = torch.empty((int(L.fgx_narrow_plan_bytes(nat.sz(n), C.c_int(27))),), dtype=torch.uint8, device=gpu_device)
    sched = nat.table_lookup(nat.PASS_FWD, torch.float16, n, c, c, 27)
    outs = []
    with torch.cuda.device(gpu_device):
        panel = impl._weight_panel(None, wd.contiguous(), nat.DTYPE_CODE[torch.float16], 0, sched, gpu_device)
        for same_rows in (1, 0):
            nat.check(L.fgx_narrow_plan(nat.ptr(nmap), nat.ptr(order), nat.sz(n), C.c_int(27), C.c_int(same_rows), nat.ptr(plan), nat.stream()))
            o = torch.empty((n, c), dtype=torch.float16, device=gpu_device)
            nat.check(L.fgx_conv_narrow_gemm(C.c_int(nat.DTYPE_CODE[torch.float16]), nat.ptr(fd), nat.ptr(panel), nat.ptr(bd), nat.ptr(nmap),
                                             nat.ptr(plan), nat.sz(n), nat.sz(n), C.c_int(c), C.c_int(c), C.c_int(27), C.c_int(nat.ACT_RELU),
                                             nat.ptr(o), nat.ptr(None), nat.stream()))
            outs.append(o.cpu())
            chunks = -(-n // 128)
            raw = plan.cpu().numpy()
            table = raw[256:].reshape(chunks, 8192 + 448 * 4 + 512)[:, :8192].copy().view(np.uint16).reshape(chunks, 128, 32)
            assert (table[:, :, 31] != 0).any(), "no chunk overflowed: the test does not reach the path it is for"
            assert int(raw[:4].view(np.uint32)[0]) == int((table[:, :, 31] != 0).any(1).sum()), "the header does not count the overflowing chunks"
    assert torch.equal(outs[0], out.cpu()) and torch.equal(outs[1], out.cpu())


@pytest.mark.parametrize("res", [1, 2, 4])
def test_degenerate_sizes(gpu_device, res):
    # fewer voxels than one tile; N = 1 at res 1
    _say(f"conv degenerate res={res}")
    coords_np = reference_test_shell(res)
    for dtype in (torch.float16, torch.float32):
        _run_and_check(coords_np, torch.Size([1, 64, res, res, res]), 64, 64, dtype, gpu_device, seed=res)


def test_empty_input_through_the_operator(gpu_device):
    """No voxel at all: an empty output, and a backward pass that returns an empty input gradient and zero weight and bias
    gradients -- both schedules, the resident-row kernels on "auto" and forced on, channel counts that need padding."""
    from flex_gemm.ops.spconv import set_algorithm, sparse_submanifold_conv3d_relu
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    old = impl.spconv.NARROW_RESIDENT
    try:
        for algo in (Algorithm.MASKED_IMPLICIT_GEMM_SPLITK, Algorithm.IMPLICIT_GEMM):
            set_algorithm(algo)
            for narrow in ("auto", "on"):
                impl.spconv.NARROW_RESIDENT = narrow
                for dt, c in ((torch.float16, 32), (torch.float32, 64), (torch.bfloat16, 20)):
                    _say(f"conv of an empty input {algo} narrow={narrow} {dt} C={c}")
                    coords = torch.zeros((0, 4), dtype=torch.int32, device=gpu_device)
                    f = torch.zeros((0, c), dtype=dt, device=gpu_device, requires_grad=True)
                    w = torch.randn(c, 3, 3, 3, c, device=gpu_device).to(dt).requires_grad_(True)
                    b = torch.randn(c, device=gpu_device).to(dt).requires_grad_(True)
                    for op in (sparse_submanifold_conv3d, sparse_submanifold_conv3d_relu):
                        f.grad = w.grad = b.grad = None
                        out, _ = op(f, coords, torch.Size([1, c, 8, 8, 8]), w, b)
                        assert out.shape == (0, c) and out.dtype == dt
                        out.backward(torch.zeros_like(out))
                        torch.cuda.synchronize()
                        assert f.grad.shape == (0, c)
                        assert w.grad.shape == w.shape and float(w.grad.abs().max()) == 0.0
                        assert b.grad.shape == b.shape and float(b.grad.abs().max()) == 0.0
    finally:
        impl.spconv.NARROW_RESIDENT = old
        set_algorithm(Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("dtype,ci,co,res", [(torch.float16, 64, 32, 24), (torch.float32, 5, 7, 16), (torch.bfloat16, 128, 128, 32),
                                             (torch.float16, 24, 16, 48)])
def test_strided_views_and_partial_gradients(gpu_device, dtype, ci, co, res, relu):
    """Arguments that are views with strides of their own -- the weight a permuted [Ci, Kw, Kh, Kd, Co] tensor, the bias
    a column of a matrix, the upstream gradient a transposed tensor -- give the bits of their dense copies; so do calls
    where only the weight, or only the features, want a gradient, and a call without bias."""
    from flex_gemm.ops.spconv import sparse_submanifold_conv3d_relu
    op = sparse_submanifold_conv3d_relu if relu else sparse_submanifold_conv3d
    _say(f"strided views {dtype} ci={ci} co={co} res={res} relu={relu}")
    dev = gpu_device
    coords = torch.from_numpy(reference_test_shell(res)).to(dev)
    n = coords.shape[0]
    shape = torch.Size([1, ci, res, res, res])
    g = torch.Generator().manual_seed(1)
    f0 = torch.randn(n, ci, generator=g).to(dtype).to(dev)
    w0 = (torch.randn(co, 3, 3, 3, ci, generator=g) / (27 * ci) ** 0.5).to(dtype).to(dev)
    b0 = torch.randn(co, generator=g).to(dtype).to(dev)
    go0 = torch.randn(n, co, generator=g).to(dtype).to(dev)

    def step(f, w, b, go):
        out = op(f, coords, shape, w, b)[0]
        out.backward(go)
        torch.cuda.synchronize()
        return out.detach()

    f, w, b = f0.clone().requires_grad_(True), w0.clone().requires_grad_(True), b0.clone().requires_grad_(True)
    ref = (step(f, w, b, go0), f.grad, w.grad, b.grad)
    ws = w0.permute(4, 1, 2, 3, 0).contiguous().permute(4, 1, 2, 3, 0).requires_grad_(True)
    bs = torch.stack([b0, b0], 1)[:, 0].requires_grad_(True)
    gos = go0.t().contiguous().t()
    assert not ws.is_contiguous() and not bs.is_contiguous() and not gos.is_contiguous()
    f = f0.clone().requires_grad_(True)
    out = step(f, ws, bs, gos)
    for name, a, r in zip(("output", "input gradient", "weight gradient", "bias gradient"), (out, f.grad, ws.grad, bs.grad), ref):
        assert a.shape == r.shape and torch.equal(a, r), name
    w = w0.clone().requires_grad_(True)                         # only the weight wants a gradient
    assert torch.equal(step(f0, w, b0, go0), ref[0]) and torch.equal(w.grad, ref[2])
    f = f0.clone().requires_grad_(True)                         # only the features do
    assert torch.equal(step(f, w0, b0, go0), ref[0]) and torch.equal(f.grad, ref[1])
    if not relu:                                                # no bias: the gradients do not depend on it
        f, w = f0.clone().requires_grad_(True), w0.clone().requires_grad_(True)
        out = step(f, w, None, go0)
        assert torch.equal(f.grad, ref[1]) and torch.equal(w.grad, ref[2])
        tol = 1e-4 if dtype == torch.float32 else 1e-2
        assert float((out.float() + b0.float() - ref[0].float()).abs().max() / ref[0].float().abs().max()) < tol


def test_odd_channel_counts_batches_dilation_no_bias(gpu_device):
    rng = np.random.default_rng(3)
    res = 12
    coords_np = reference_test_shell(res, batch=2)
    coords_np = coords_np[rng.permutation(len(coords_np))]
    shape = torch.Size([2, 0, res, res, res])
    for ci, co, dtype in [(5, 7, torch.float32), (20, 12, torch.float16), (48, 96, torch.bfloat16), (3, 130, torch.float16)]:
        _say(f"conv odd channels ci={ci} co={co} {dtype}")
        _run_and_check(coords_np, shape, ci, co, dtype, gpu_device, seed=ci, dilation=(2, 1, 1), use_bias=False)
    _say("conv 1x3x3 kernel")
    _run_and_check(coords_np, shape, 32, 32, torch.float16, gpu_device, seed=1, ksize=(1, 3, 3))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("ci,co", [(1, 1), (1, 3), (3, 1), (2, 130), (130, 2), (257, 9), (9, 520), (1032, 17)])
def test_extreme_channel_counts(gpu_device, dtype, ci, co):
    """Single channels, rows shorter than one 16-byte chunk, and counts just past a tile (129-130, 257, 520, 1032) on
    either side, both masked and unmasked schedules."""
    res = 14
    coords_np = reference_test_shell(res)
    for algo in (Algorithm.MASKED_IMPLICIT_GEMM_SPLITK, Algorithm.IMPLICIT_GEMM):
        _say(f"conv extreme channels ci={ci} co={co} {dtype} {algo}")
        _run_and_check(coords_np, torch.Size([1, ci, res, res, res]), ci, co, dtype, gpu_device, seed=ci + co, algo=algo)


@pytest.mark.parametrize("c,dtype", [(64, torch.float16), (128, torch.bfloat16), (40, torch.float32)])
@pytest.mark.parametrize("ksize,dilation", [((5, 5, 1), (1, 1, 1)), ((1, 1, 31), (1, 1, 1)), ((1, 1, 1), (1, 1, 1)), ((3, 1, 3), (1, 2, 3)),
                                            ((1, 3, 9), (2, 1, 1)), ((1, 1, 5), (1, 1, 4))])
def test_kernel_volumes_from_1_to_32_on_wide_layers(gpu_device, c, dtype, ksize, dilation):
    """Kernel volumes other than 27 -- one offset, 31 offsets (the largest odd volume a 32-bit mask code holds) -- with and
    without dilation, on layers the streaming and sweep kernels serve.  Even extents are refused: the reference's map
    builder mirrors offset v onto V - 1 - v (subm_neighbor_map.cu:53-60), which only an odd kernel allows."""
    res = 20
    _say(f"conv ksize={ksize} dilation={dilation} c={c} {dtype}")
    coords_np = reference_test_shell(res, batch=2)
    _run_and_check(coords_np, torch.Size([2, c, res, res, res]), c, c, dtype, gpu_device, seed=c + ksize[0], ksize=ksize,
                   dilation=dilation)
    with pytest.raises(ValueError, match="odd"):
        SubMConv3dFunction._compute_neighbor_cache(torch.from_numpy(coords_np).to(gpu_device), torch.Size([2, c, res, res, res]),
                                                   (2, 3, 3), (1, 1, 1), True)


@pytest.mark.parametrize("res,c", [(512, 32), (256, 128)])
def test_whole_path_on_a_stream_of_the_caller_s_while_the_default_stream_is_busy(gpu_device, res, c):
    """Cache build (at a million voxels: map, then mask sort and pair lists side by side on two streams), forward and
    backward enqueued on a stream of the caller's, the default stream kept busy with unrelated products and no device-wide
    wait in between: the bits of the same calls on the default stream."""
    _say(f"whole path on a caller's stream, res={res} c={c}")
    dev = gpu_device
    coords = torch.from_numpy(reference_test_shell(res)).to(dev)
    n = coords.shape[0]
    shape = torch.Size([1, c, res, res, res])
    g = torch.Generator().manual_seed(res)
    f0 = torch.randn(n, c, generator=g).half().to(dev)
    w0 = (torch.randn(c, 3, 3, 3, c, generator=g) / (27 * c) ** 0.5).half().to(dev)
    b0 = torch.randn(c, generator=g).half().to(dev)
    go = torch.randn(n, c, generator=g).half().to(dev)

    def steps(count):
        got = []
        for _ in range(count):
            f, w, b = f0.clone().requires_grad_(True), w0.clone().requires_grad_(True), b0.clone().requires_grad_(True)
            cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
            h = sparse_submanifold_conv3d(f, coords, shape, w, b, cache)[0]
            h = sparse_submanifold_conv3d(h, coords, shape, w, b, cache)[0]
            h.backward(go)
            got.append((h.detach(), f.grad, w.grad, b.grad, cache.neighbor_map, cache.sorted_idx, cache.valid_signal_i))
        return got

    ref = steps(1)[0]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    busy = torch.randn(4096, 4096, device=dev)
    side.wait_stream(torch.cuda.current_stream())
    for _ in range(20):
        busy = torch.tanh(busy @ busy) * 0.5
    with torch.cuda.stream(side):
        got = steps(3)
    for _ in range(20):
        busy = torch.tanh(busy @ busy) * 0.5
    side.synchronize()
    torch.cuda.synchronize()
    for one in got:
        for name, a, r in zip(("output", "input gradient", "weight gradient", "bias gradient", "map", "order", "pairs"), one, ref):
            assert torch.equal(a, r), name


@pytest.mark.parametrize("needs_grad", [True, False])
def test_one_cache_serves_layers_of_any_type_width_and_schedule(gpu_device, needs_grad):
    """One neighbor cache (built with or without the gradient tables: a backward pass makes them when they are missing)
    serves fp16, fp32 and bf16 layers of different widths under the masked and the unmasked schedule, one after the
    other; every product and gradient has the bits a fresh cache gives.  The tables a cache keeps per shape (work lists,
    sweep plans, tile orders) must not leak from one layer shape or type into the next."""
    from flex_gemm.ops.spconv import set_algorithm
    dev = gpu_device
    res = 128
    coords = torch.from_numpy(reference_test_shell(res)).to(dev)
    n = coords.shape[0]
    shape = torch.Size([1, 1, res, res, res])
    masked, plain = Algorithm.MASKED_IMPLICIT_GEMM_SPLITK, Algorithm.IMPLICIT_GEMM
    layers = [(torch.float16, 128, 128, masked), (torch.float32, 128, 128, masked), (torch.bfloat16, 64, 64, masked),
              (torch.float16, 128, 256, masked), (torch.float16, 256, 128, plain), (torch.float16, 128, 128, plain),
              (torch.bfloat16, 128, 128, masked), (torch.float32, 40, 72, masked), (torch.float16, 1024, 64, masked),
              (torch.float16, 64, 1024, masked), (torch.float16, 128, 128, masked)]

    def step(tensors, cache, algo):
        set_algorithm(algo)
        f, w, b = (t.clone().requires_grad_(True) for t in tensors[:3])
        out = sparse_submanifold_conv3d(f, coords, shape, w, b, cache)[0]
        out.backward(tensors[3])
        torch.cuda.synchronize()
        return out.detach(), f.grad, w.grad, b.grad

    try:
        shared = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), needs_grad)
        for i, (dt, ci, co, algo) in enumerate(layers):
            _say(f"shared cache, layer {i}: {dt} {ci}->{co} {algo}")
            tensors = tuple(t.to(dev) for t in _case(np.empty((n, 4)), ci, co, dt, seed=i))
            got = step(tensors, shared, algo)
            ref = step(tensors, SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True), algo)
            for name, a, r in zip(("output", "input gradient", "weight gradient", "bias gradient"), got, ref):
                assert torch.equal(a, r), (i, name)
    finally:
        set_algorithm(masked)


def test_four_host_threads_call_the_library_at_once(gpu_device):
    """ctypes drops the interpreter lock around a foreign call, so threads of one process are inside the library together.
    Four threads, each on a stream of its own and with a layer shape of its own, build caches and run forward and
    backward a few times over; every thread gets the bits the same calls give when they run alone."""
    import threading
    dev = gpu_device
    cases = [(48, 128, 128, torch.float16), (40, 32, 32, torch.bfloat16), (32, 64, 256, torch.float16), (24, 40, 72, torch.float32)]

    def work(res, ci, co, dt, rounds):
        coords = torch.from_numpy(reference_test_shell(res)).to(dev)
        shape = torch.Size([1, ci, res, res, res])
        tensors = [t.to(dev) for t in _case(np.empty((coords.shape[0], 4)), ci, co, dt, seed=res)]
        got = []
        for _ in range(rounds):
            f, w, b = (t.clone().requires_grad_(True) for t in tensors[:3])
            out, cache = sparse_submanifold_conv3d(f, coords, shape, w, b)
            out.backward(tensors[3])
            got.append((out.detach(), f.grad, w.grad, b.grad, cache.sorted_idx))
        torch.cuda.current_stream().synchronize()
        return got

    alone = [work(*case, 1)[0] for case in cases]
    torch.cuda.synchronize()
    results, errors = [None] * len(cases), []

    def thread_main(i):
        try:
            with torch.cuda.stream(torch.cuda.Stream()):
                results[i] = work(*cases[i], 6)
        except BaseException as e:              # reported by the main thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=thread_main, args=(i,)) for i in range(len(cases))]
    _say("four threads inside the library")
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a thread did not finish"
    assert not errors, errors
    torch.cuda.synchronize()
    for i, rounds in enumerate(results):
        for got in rounds:
            for name, a, r in zip(("output", "input gradient", "weight gradient", "bias gradient", "order"), got, alone[i]):
                assert torch.equal(a, r), (cases[i], name)


@pytest.mark.parametrize("mode", ["no_grad", "inference_mode"])
def test_calls_that_record_no_gradients_build_no_gradient_tables(gpu_device, mode):
    """Under torch.no_grad() / inference_mode() the weights still say requires_grad, but no backward pass can follow: the
    cache such a call builds carries no pair lists, the fused ReLU writes no bit mask, and the results are those of a
    recording call.  A cache made that way still serves a later training step (its tables are made when asked for)."""
    from flex_gemm.ops.spconv import sparse_conv3d, sparse_submanifold_conv3d_relu
    dev = gpu_device
    res, c = 32, 64
    _say(f"calls under {mode}")
    coords = torch.from_numpy(reference_test_shell(res)).to(dev)
    shape = torch.Size([1, c, res, res, res])
    f, w, b, go = (t.to(dev) for t in _case(np.empty((coords.shape[0], 4)), c, c, torch.float16, seed=4))
    w, b = torch.nn.Parameter(w), torch.nn.Parameter(b)
    ref, trained = sparse_submanifold_conv3d(f, coords, shape, w, b)
    assert hasattr(trained, "valid_signal_i")
    with getattr(torch, mode)():
        out, lean = sparse_submanifold_conv3d(f, coords, shape, w, b)
        assert torch.equal(out, ref) and not out.requires_grad
        assert not hasattr(lean, "valid_signal_i"), "gradient tables were built for a call that cannot use them"
        assert torch.equal(sparse_submanifold_conv3d(f, coords, shape, w, b, trained)[0], ref)
        assert torch.equal(sparse_submanifold_conv3d_relu(f, coords, shape, w, b, lean)[0], torch.relu(ref))
        _, _, lean_generic = sparse_conv3d(f, coords, shape, w, b, stride=(2, 2, 2), padding=(1, 1, 1))
        assert not hasattr(lean_generic, "valid_signal_i")
    grads = []
    for cache in (trained, lean):
        f2 = f.clone().requires_grad_(True)
        w.grad = b.grad = None
        sparse_submanifold_conv3d(f2, coords, shape, w, b, cache)[0].backward(go)
        grads.append((f2.grad, w.grad, b.grad))
    assert all(torch.equal(a, r) for a, r in zip(grads[1], grads[0]))


def test_algorithm_values_and_cache_reuse(gpu_device):
    res, c = 16, 64
    coords_np = reference_test_shell(res)
    shape = torch.Size([1, c, res, res, res])
    cache = None
    for algo in (Algorithm.MASKED_IMPLICIT_GEMM_SPLITK, Algorithm.MASKED_IMPLICIT_GEMM, Algorithm.IMPLICIT_GEMM,
                 Algorithm.IMPLICIT_GEMM_SPLITK, Algorithm.EXPLICIT_GEMM):
        _say(f"conv algorithm {algo}")
        cache, _ = _run_and_check(coords_np, shape, c, c, torch.float16, gpu_device, seed=5, algo=algo, cache=cache)
    # a cache built without gradients (inference) is completed on demand when a training step reuses it
    _say("inference cache reused for training")
    coords = torch.from_numpy(coords_np).to(gpu_device)
    inf_cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), False)
    assert not hasattr(inf_cache, "valid_signal_i")
    _run_and_check(coords_np, shape, c, c, torch.float16, gpu_device, seed=6, cache=inf_cache)
    # under no_grad the operator builds the inference cache itself
    with torch.no_grad():
        f, w, b, _ = _case(coords_np, c, c, torch.float16, 7)
        out, cch = sparse_submanifold_conv3d(f.to(gpu_device), coords, shape, w.to(gpu_device), b.to(gpu_device))
    assert not hasattr(cch, "valid_signal_i") and out.shape == (len(coords_np), c)


@pytest.mark.parametrize("stream", [0, 1])
def test_non_masked_schedule(gpu_device, stream):
    """IMPLICIT_GEMM[_SPLITK]: the cache is the neighbor map alone (reference submanifold_conv3d.py:59-71) and the
    kernels walk the natural row order with all 27 offsets per tile; same results as the oracle."""
    res, c = 24, 128
    coords_np = reference_test_shell(res)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([1, c, res, res, res])
    for algo in (Algorithm.IMPLICIT_GEMM, Algorithm.IMPLICIT_GEMM_SPLITK):
        _say(f"non-masked schedule {algo} stream={stream}")
        flex_gemm.ops.spconv.set_algorithm(algo)
        try:
            cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
        finally:
            flex_gemm.ops.spconv.set_algorithm(Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)
        assert [k for k in vars(cache) if not k.startswith("_")] == ["neighbor_map"]
        fields = dict(tile_rows=256, tile_cols=128, slab_bytes=128, splitk=1, stream=1) if stream else dict(stream=0)
        with _force_schedule(**fields):
            _run_and_check(coords_np, shape, c, c, torch.float16, gpu_device, seed=41, algo=algo, cache=cache)
        assert hasattr(cache, "_dense_order") and (stream == 0 or hasattr(cache, "_plan_d_256"))


def test_private_row_order_is_used_and_equivalent(gpu_device):
    """Short rows (<= 128 bytes) of a large enough map run on the Z-order-chunked private row order once the cache has
    served a few passes on the public one, long rows always on the public mask-sorted order; both give the oracle's result
    (checked by _run_and_check) and agree with each other."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    res = 24
    coords_np = reference_test_shell(res)
    coords_np = coords_np[np.random.default_rng(0).permutation(len(coords_np))]
    shape = torch.Size([1, 0, res, res, res])
    old = (impl.LOCALITY_MAX_ROW_BYTES, impl.LOCALITY_MIN_ROWS, impl.LOCALITY_AFTER_CALLS)
    try:
        _say("private row order: a small map stays on the public order")
        cache0, _ = _run_and_check(coords_np, shape, 32, 32, torch.float16, gpu_device, seed=20)
        assert not hasattr(cache0, "_tile_order")
        impl.LOCALITY_MIN_ROWS, impl.LOCALITY_AFTER_CALLS = 0, 0
        _say("private row order: C=32 fp16 (64-byte rows)")
        cache, _ = _run_and_check(coords_np, shape, 32, 32, torch.float16, gpu_device, seed=21)
        assert hasattr(cache, "_tile_order")
        _say("public row order: C=128 fp16 (256-byte rows)")
        cache2, _ = _run_and_check(coords_np, shape, 128, 128, torch.float16, gpu_device, seed=22)
        assert not hasattr(cache2, "_tile_order")
        f, w, b, _ = _case(coords_np, 32, 32, torch.float16, 23)
        f, w, b = f.to(gpu_device), w.to(gpu_device).reshape(32, 27, 32), b.to(gpu_device)
        outs = []
        for limit in (0, 1 << 20):
            impl.LOCALITY_MAX_ROW_BYTES = limit
            fresh = SubMConv3dFunction._compute_neighbor_cache(torch.from_numpy(coords_np).to(gpu_device), shape, (3, 3, 3), (1, 1, 1), False)
            outs.append(impl._gather_gemm(f, w, b, fresh, 0, True).float().cpu())
            assert hasattr(fresh, "_tile_order") == (limit > 0)
        assert eg.max_rel_err(outs[0], outs[1].double()) <= 2e-3
        # the order comes when the cache has served LOCALITY_AFTER_CALLS short-row passes on the public one, and changes
        # no result beyond the rounding of a different tile split
        _say("private row order: made at the third pass of a cache")
        impl.LOCALITY_MAX_ROW_BYTES, impl.LOCALITY_AFTER_CALLS = old[0], 2
        late = SubMConv3dFunction._compute_neighbor_cache(torch.from_numpy(coords_np).to(gpu_device), shape, (3, 3, 3), (1, 1, 1), False)
        seen = []
        for call in range(4):
            seen.append(impl._gather_gemm(f, w, b, late, 0, True).float().cpu())
            assert hasattr(late, "_tile_order") == (call >= 2), call
        assert torch.equal(seen[0], seen[1]) and torch.equal(seen[2], seen[3])
        assert eg.max_rel_err(seen[0], seen[2].double()) <= 2e-3
    finally:
        impl.LOCALITY_MAX_ROW_BYTES, impl.LOCALITY_MIN_ROWS, impl.LOCALITY_AFTER_CALLS = old


@pytest.mark.parametrize("res,chans,iterations", [(128, (16, 32, 64, 32, 16, 8), 5), (512, (32, 16, 32, 64, 24), 3)])
def test_kernel_choice_over_a_cache_s_life_keeps_the_results(gpu_device, res, chans, iterations):
    """Layers of different widths share one cache over several training iterations, the policies left on "auto": the
    cache's first products run on the streaming kernels, later ones on the resident-row kernels once it has earned
    their plan (64 160 voxels: after sixteen products; 1 026 536 voxels: from the second product on).  Every iteration's
    output and gradients stay within fp16 rounding of the first iteration's, and iterations after the switch agree bit
    for bit.  The upstream gradient has stride 0, as out.sum().backward() makes it (scaled by 2^-10: a million ones would
    overflow an fp16 bias gradient)."""
    _say(f"kernel choice over a cache's life, res={res} widths={chans}")
    dev = gpu_device
    coords = torch.from_numpy(reference_test_shell(res)).to(dev)
    n = coords.shape[0]
    g = torch.Generator().manual_seed(res)
    feats = torch.randn(n, chans[0], generator=g).half().to(dev).requires_grad_(True)
    params = [((torch.randn(co, 3, 3, 3, ci, generator=g) / (27 * ci) ** 0.5).half().to(dev).requires_grad_(True),
               torch.randn(co, generator=g).half().to(dev).requires_grad_(True)) for ci, co in zip(chans[:-1], chans[1:])]
    shape = torch.Size([1, chans[0], res, res, res])
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    results = []
    for it in range(iterations):
        feats.grad = None
        for w, b in params:
            w.grad = None
            b.grad = None
        h = feats
        for w, b in params:
            h = sparse_submanifold_conv3d(h, coords, shape, w, b, cache)[0]
        (h.sum() * 2.0 ** -10).backward()
        torch.cuda.synchronize()
        results.append([h.detach().clone(), feats.grad.clone()] + [w.grad.clone() for w, _ in params] + [b.grad.clone() for _, b in params])
    assert hasattr(cache, "_narrow_plan_buf"), "the cache never earned the resident-row plan"
    assert all(bool(torch.isfinite(r).all()) for r in results[0])
    for got in results[1:]:
        for a, r in zip(got, results[0]):
            assert float((a.float() - r.float()).abs().max() / r.float().abs().max().clamp_min(1e-6)) < 2e-3
    assert all(torch.equal(a, r) for a, r in zip(results[-1], results[-2]))


def test_forced_splitk_matches_unsplit(gpu_device):
    """Split-K partial sums add up to the unsplit result (fp32 rounding apart)."""
    import ctypes as C
    from flexgemm_amd import _native as nat
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    res, c = 16, 128
    _say("forced split-K")
    coords_np = reference_test_shell(res)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([1, c, res, res, res])
    f, w, b, _ = _case(coords_np, c, c, torch.float16, 9)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), False)
    outs = []
    real = nat.table_lookup
    for s in (1, 2, 5):
        def forced(*a, _s=s):
            sc = real(*a)
            sc.splitk = _s
            return sc
        nat.table_lookup = forced
        try:
            outs.append(impl._gather_gemm(f.to(gpu_device), w.to(gpu_device).reshape(c, 27, c), b.to(gpu_device), cache, 0, True).float().cpu())
        finally:
            nat.table_lookup = real
    assert eg.max_rel_err(outs[1], outs[0].double()) <= 2e-3 and eg.max_rel_err(outs[2], outs[0].double()) <= 2e-3


def _force_schedule(wgrad=False, **fields):
    """Context manager: fwd/dgrad (or, with wgrad=True, wgrad) schedules from the table with the given fields overridden."""
    import contextlib
    from flexgemm_amd import _native as nat

    @contextlib.contextmanager
    def cm():
        real = nat.table_lookup

        def forced(pass_kind, *a):
            sc = real(pass_kind, *a)
            if (pass_kind == nat.PASS_WGRAD) == wgrad:
                for k, v in fields.items():
                    setattr(sc, k, v)
            return sc
        nat.table_lookup = forced
        try:
            yield
        finally:
            nat.table_lookup = real
    return cm()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("res,ci,co", [(32, 128, 128), (24, 64, 256), (24, 96, 40), (16, 8, 136), (48, 256, 128)])
def test_streaming_kernel_matches_oracle(gpu_device, dtype, res, ci, co):
    """Forward, dgrad (and the untouched wgrad) with the persistent streaming GEMM forced: several column tiles,
    contraction widths that are not whole K-slabs, fewer tiles than workgroups, rows past the last tile."""
    _say(f"stream res={res} ci={ci} co={co} {dtype}")
    coords_np = reference_test_shell(res)
    shape = torch.Size([1, ci, res, res, res])
    with _force_schedule(tile_rows=256, tile_cols=128, slab_bytes=128, splitk=1, stream=1):
        _run_and_check(coords_np, shape, ci, co, dtype, gpu_device, seed=21)
    if co <= 136:   # the narrow-tile variant of the streaming kernel (64 columns per tile)
        with _force_schedule(tile_rows=256, tile_cols=64, slab_bytes=128, splitk=1, stream=1):
            _run_and_check(coords_np, shape, ci, co, dtype, gpu_device, seed=22)
    # the wide-tile variant (128 rows x 256 columns: 2 x 4 multipliers), also where most of its columns are padding
    with _force_schedule(tile_rows=128, tile_cols=256, slab_bytes=128, splitk=1, stream=1):
        cache, _ = _run_and_check(coords_np, shape, ci, co, dtype, gpu_device, seed=24)
    assert any(k.startswith("_plan_") and k.endswith("_128") for k in vars(cache)), "the 128-row gather plan was not used"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("res,ci,co,tile_cols", [(32, 32, 32, 32), (24, 32, 64, 64), (24, 16, 96, 128), (24, 128, 40, 32),
                                                 (16, 24, 32, 32), (40, 32, 32, 32)])
def test_streaming_kernel_with_64_byte_slabs(gpu_device, dtype, res, ci, co, tile_cols):
    """The streaming GEMM on 64-byte K-slabs (rows shorter than 128 bytes) with 32-, 64- and 128-column tiles: panels
    narrower than one round of loader instructions, several slabs per row, ragged last slabs, several column tiles."""
    _say(f"stream slab64 res={res} ci={ci} co={co} tile_cols={tile_cols} {dtype}")
    coords_np = reference_test_shell(res)
    shape = torch.Size([1, ci, res, res, res])
    with _force_schedule(tile_rows=256, tile_cols=tile_cols, slab_bytes=64, splitk=1, stream=1):
        _run_and_check(coords_np, shape, ci, co, dtype, gpu_device, seed=29)


def test_streaming_kernel_equals_tiled_kernel_bitwise(gpu_device):
    """Both kernels add the same products in the same order (offsets ascending, K ascending), so their outputs
    agree bit for bit; isolated voxels (only the centre offset) and a batch dimension are in the mix."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    _say("stream vs tiled, bitwise")
    res, c = 40, 128
    shell = reference_test_shell(res)
    rng = np.random.default_rng(5)
    lonely = np.stack([np.zeros(40, np.int32), rng.integers(0, 4, 40), rng.integers(0, 4, 40), rng.integers(0, 4, 40)], 1).astype(np.int32) * 9
    lonely = lonely[np.unique(lonely, axis=0, return_index=True)[1]]
    second = shell.copy()
    second[:, 0] = 1
    coords_np = np.concatenate([shell, second, lonely + np.array([2, 0, 0, 0], np.int32)], 0).astype(np.int32)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([3, c, res, res, res])
    f, w, b, g = _case(coords_np, c, c, torch.float16, 31)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    outs = []
    for stream in (0, 1):
        fields = dict(tile_rows=256, tile_cols=128, slab_bytes=128, splitk=1, stream=1) if stream else \
            dict(tile_rows=128, tile_cols=128, slab_bytes=64, splitk=1, stream=0)
        with _force_schedule(**fields):
            o = impl._gather_gemm(f.to(gpu_device), w.to(gpu_device).reshape(c, 27, c), b.to(gpu_device), cache, 0, False)
            gi = impl._gather_gemm(g.to(gpu_device), w.to(gpu_device).reshape(c, 27, c), None, cache, 1, False)
        outs.append((o.cpu(), gi.cpu()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("res,ci,co,block_rows", [(48, 128, 128, 0), (48, 128, 128, 2048), (48, 32, 32, 0), (40, 64, 256, 1024),
                                                   (40, 256, 64, 0), (64, 64, 64, 4096), (24, 128, 128, 0)])
def test_bias_gradient_rides_along_with_wgrad(gpu_device, dtype, res, ci, co, block_rows):
    """dbias from the streaming wgrad kernel (grad_out rows of the centre offset times a fragment of ones): equal to the
    column sums within the operator's tolerance, for wide, narrow (pairs split over the multipliers), multi-tile and
    single-block shapes, and the weight gradient itself is unchanged bit for bit.  The last shape is below the streaming
    range: there the call falls back to the stand-alone column sum."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    _say(f"fused dbias res={res} ci={ci} co={co} block_rows={block_rows} {dtype}")
    coords_np = reference_test_shell(res)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    f, w, b, g = _case(coords_np, ci, co, dtype, 53)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, torch.Size([1, ci, res, res, res]), (3, 3, 3), (1, 1, 1), True)
    fields = dict(block_rows=block_rows) if block_rows else {}
    with _force_schedule(wgrad=True, **fields):
        gw_plain = impl._wgrad(g.to(gpu_device), f.to(gpu_device), cache, 27)
        gw, gb = impl._wgrad(g.to(gpu_device), f.to(gpu_device), cache, 27, True, 13)
        gw2, gb2 = impl._wgrad(g.to(gpu_device), f.to(gpu_device), cache, 27, True, -1)       # no such offset: column sum
    assert torch.equal(gw, gw_plain) and torch.equal(gw2, gw_plain)
    ref = g.double().sum(0)
    assert gb.dtype == dtype and gb.shape == (co,)
    assert eg.max_rel_err(gb.cpu(), ref) <= TOL[dtype]
    assert eg.max_rel_err(gb2.cpu(), ref) <= TOL[dtype]
    assert torch.equal(gb2, impl._colsum(g.to(gpu_device)))


def test_item_order_changes_nothing(gpu_device):
    """How the streaming GEMM's tiles are dealt to its workgroups is a scheduling choice: every order gives the same
    bits (more items than resident workgroups, two column tiles per row tile)."""
    import flex_gemm
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    res, ci, co = 192, 64, 256
    coords_np = reference_test_shell(res)
    assert -(-len(coords_np) // 256) * 2 > 256               # more than one round of items: the dealt order is used
    _say(f"item orders res={res} n={len(coords_np)}")
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([1, ci, res, res, res])
    f, w, b, g = _case(coords_np, ci, co, torch.float16, 41)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    outs = {}
    try:
        for mode in ("default", "balanced", "auto"):
            flex_gemm.ops.spconv.GEMM_ITEM_ORDER = mode
            with _force_schedule(tile_rows=256, tile_cols=128, slab_bytes=128, splitk=1, stream=1):
                outs[mode] = impl._gather_gemm(f.to(gpu_device), w.to(gpu_device).reshape(co, 27, ci), b.to(gpu_device), cache, 0,
                                               False).cpu()
    finally:
        flex_gemm.ops.spconv.GEMM_ITEM_ORDER = "auto"
    assert any(k.startswith("_items_") for k in vars(cache))
    for mode in ("balanced", "auto"):
        assert torch.equal(outs[mode], outs["default"]), mode
    rows = torch.from_numpy(np.random.default_rng(3).choice(len(coords_np), 4000, replace=False))
    ref_rows = eg.forward(f.double(), cache.neighbor_map.cpu().view(torch.int32)[rows], w.double(), b.double())
    assert eg.max_rel_err(outs["default"][rows], ref_rows) <= 1e-2          # fp16 tolerance


def _load_spread(item_at, codes, col_tiles, groups, slabs):
    """busiest workgroup / mean, with the cost model of the ordering kernel"""
    offsets = np.array([bin(int(c)).count("1") for c in codes])
    cost = np.maximum(offsets, 1) * slabs + 3
    load = np.zeros(groups)
    np.add.at(load, np.arange(len(item_at)) % groups, cost[np.asarray(item_at) // col_tiles])
    return load.max() / load.mean()


def test_item_order_evens_out_the_benchmark_shell(gpu_device):
    """At the res-512 benchmark shape (2615 tiles of 256 rows for 256 workgroups) the kernel's own round-robin leaves the
    busiest workgroup ~17 % above the mean; the dealt order brings it within 3 % (within 10 % when there are only five rounds of items)."""
    from flexgemm_amd.workloads import shell_coords
    res = 512
    coords = torch.from_numpy(shell_coords(res)).to(gpu_device)
    _say(f"item order at res {res}, n={coords.shape[0]}")
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, torch.Size([1, 128, res, res, res]), (3, 3, 3), (1, 1, 1), False)
    import flex_gemm
    _, code, _, _, _, key = cache._gather_plan(256, False)
    for col_tiles, groups, slabs in ((1, 256, 2), (2, 256, 4), (1, 512, 1)):
        flex_gemm.ops.spconv.GEMM_ITEM_ORDER = "balanced"       # ("auto" deals rows of 512 bytes and more only)
        try:
            item_at = cache._item_order(key, code, col_tiles, groups, slabs).cpu().numpy().astype(np.int64)
        finally:
            flex_gemm.ops.spconv.GEMM_ITEM_ORDER = "auto"
        codes = code.cpu().numpy().view(np.uint32)
        total = col_tiles * len(codes)
        assert sorted(item_at.tolist()) == list(range(total))
        own = _load_spread(np.arange(total - 1, -1, -1), codes, col_tiles, groups, slabs)
        dealt = _load_spread(item_at, codes, col_tiles, groups, slabs)
        _say(f"  col_tiles={col_tiles} groups={groups}: busiest/mean {own:.3f} -> {dealt:.3f}")
        assert dealt < 1.12 and dealt < own - 0.05


def test_gather_plan_band_masks(gpu_device):
    """plan_band bit b of a plan row says whether rows [32 b, 32 b + 32) of that row's index column hold a neighbor;
    the shell with scattered isolated voxels gives full, partial and (for the tail tile) sparse masks."""
    _say("gather plan band masks")
    res = 40
    shell = reference_test_shell(res)
    rng = np.random.default_rng(11)
    lonely = (np.stack([np.zeros(300, np.int32), rng.integers(0, 13, 300), rng.integers(0, 13, 300), rng.integers(0, 13, 300)], 1) * 3).astype(np.int32)
    lonely = lonely[np.unique(lonely, axis=0, return_index=True)[1]]
    lonely[:, 0] = 1
    coords_np = np.concatenate([shell, lonely], 0).astype(np.int32)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([2, 8, res, res, res])
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    for dense in (False, True):
        order, code, seg, plan_idx, plan_band, _ = cache._gather_plan(256, False, dense=dense)
        torch.cuda.synchronize()
        used = int(seg.cpu()[-1])                    # (the lists are allocated at their bound)
        assert plan_idx.shape[0] >= used and plan_band.shape[0] == plan_idx.shape[0]
        idx = plan_idx.cpu().numpy()[:used]
        got = plan_band.cpu().numpy()[:used]
        live = (idx != 0xFFFFFFFF).reshape(idx.shape[0], 8, 32).any(axis=2)
        want = (live.astype(np.uint32) << np.arange(8, dtype=np.uint32)).sum(axis=1).astype(np.uint32)
        assert np.array_equal(got, want)
        assert used == (code.shape[0] * 27 if dense else used)
        if not dense:
            assert (got != 0xFF).any() and (got == 0xFF).any()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("res,ci,co,tile,block_rows", [(32, 128, 128, 128, 1024), (24, 64, 64, 64, 512), (24, 96, 40, 128, 300),
                                                       (16, 256, 136, 128, 100000), (48, 128, 128, 128, 37),
                                                       (32, 32, 32, 32, 2048), (24, 24, 72, 32, 300), (40, 32, 32, 32, 100000),
                                                       (24, 16, 32, 32, 50)])
def test_streaming_wgrad_matches_oracle(gpu_device, dtype, res, ci, co, tile, block_rows):
    """wgrad with the persistent streaming kernel forced: edge tiles, several Co / Ci tiles, voxel blocks smaller
    than a 64-pair step (most steps partial, many empty items) and one block for everything; the 32 x 32 tile splits
    the pairs of a step over its four multiplying wavefronts (ragged steps, channel counts below the tile)."""
    _say(f"stream wgrad res={res} ci={ci} co={co} tile={tile} block_rows={block_rows} {dtype}")
    coords_np = reference_test_shell(res)
    shape = torch.Size([1, ci, res, res, res])
    with _force_schedule(wgrad=True, tile_rows=tile, tile_cols=tile, block_rows=block_rows, stream=1):
        _run_and_check(coords_np, shape, ci, co, dtype, gpu_device, seed=23)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tile", [(256, 128), (128, 256)])
@pytest.mark.parametrize("res,ci,co,block_rows", [(24, 128, 512, 1024), (16, 384, 256, 100000), (16, 256, 136, 300),
                                                  (32, 200, 264, 37), (24, 512, 96, 2048)])
def test_streaming_wgrad_with_256x128_tiles_matches_oracle(gpu_device, dtype, res, ci, co, block_rows, tile):
    """The block-major streaming wgrad kernel on 256 x 128 (Co x Ci) and 128 x 256 tiles of the weight (three ring stages of
    48 KiB, wave tiles of 128 x 64 or 64 x 128): several tiles on both sides, ragged edge tiles, one voxel block and blocks shorter than a step; with a
    bias gradient, which this tile leaves to the column-sum kernel.  Against the 128 x 128 tile the sums per element run
    over the same pairs in the same order: bit-identical."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    _say(f"stream wgrad {tile[0]}x{tile[1]} res={res} ci={ci} co={co} block_rows={block_rows} {dtype}")
    coords_np = reference_test_shell(res)
    shape = torch.Size([1, ci, res, res, res])
    with _force_schedule(wgrad=True, tile_rows=tile[0], tile_cols=tile[1], block_rows=block_rows, stream=1):
        cache, _ = _run_and_check(coords_np, shape, ci, co, dtype, gpu_device, seed=41)
    f, _, _, g = _case(coords_np, ci, co, dtype, 43)
    outs = []
    for tr, tc in (tile, (128, 128)):
        with _force_schedule(wgrad=True, tile_rows=tr, tile_cols=tc, block_rows=block_rows, stream=1):
            gw, gb = impl._wgrad(g.to(gpu_device), f.to(gpu_device), cache, 27, with_bias=True, bias_offset=13)
            outs.append((gw.cpu(), gb.cpu()))
    assert torch.equal(outs[0][0], outs[1][0]), f"{tile[0]} x {tile[1]} and 128 x 128 tiles differ"
    assert eg.max_rel_err(outs[0][1], outs[1][1].double()) <= 2e-3


@pytest.mark.parametrize("res,ci,co,tile,block_rows", [(32, 256, 256, (256, 128), 1024), (32, 256, 384, (128, 128), 4096), (28, 320, 128, (128, 256), 512),
                                                       (40, 96, 96, (64, 64), 2048), (40, 32, 24, (32, 32), 1024), (32, 1024, 512, (256, 128), 1024),
                                                       (32, 64, 64, (64, 64), 512)])
def test_streaming_wgrad_balanced_lists_change_no_bit(gpu_device, res, ci, co, tile, block_rows):
    """The streaming wgrad kernel walking the work lists that fgx_wgrad_item_lists balances by pair count against the same
    kernel on its fixed interleave: every item is summed by one workgroup in the same order and the blocks are reduced in
    the same order, so the results agree bit for bit.  The lists link every item exactly once (checked on the host), and
    lists made for another shape are ignored by the kernel."""
    import ctypes as C
    from flexgemm_amd import _native as nat
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    _say(f"stream wgrad lists res={res} ci={ci} co={co} tile={tile} block_rows={block_rows}")
    coords_np = reference_test_shell(res)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    n = coords_np.shape[0]
    shape = torch.Size([1, ci, res, res, res])
    f, _, _, g = _case(coords_np, ci, co, torch.float16, 47)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    outs = {}
    old = impl.WGRAD_BALANCED_LISTS
    try:
        for on in (False, True):
            impl.WGRAD_BALANCED_LISTS = on
            with _force_schedule(wgrad=True, tile_rows=tile[0], tile_cols=tile[1], block_rows=block_rows, stream=1):
                gw, gb = impl._wgrad(g.to(gpu_device), f.to(gpu_device), cache, 27, with_bias=True, bias_offset=13)
                outs[on] = (gw.cpu(), gb.cpu())
        lists = cache._wgrad_item_lists(block_rows, tile[0], tile[1], ci, co)
        assert lists is not None, "no lists for a shape of a few thousand items"
        w = lists.cpu().numpy().astype(np.int64)
        groups, items, tiles = int(w[0]), int(w[1]), int(w[2])
        assert tiles == -(-co // tile[0]) * -(-ci // tile[1]) and items == 27 * tiles * -(-n // block_rows) and groups % 8 == 0
        head, nxt = w[4:4 + groups], w[4 + groups:4 + groups + items]
        seen = np.zeros(items, bool)
        for h in head:
            while h != 0xFFFFFFFF:
                assert 0 <= h < items and not seen[h], "an item linked twice or out of range"
                seen[h] = True
                h = nxt[h]
        assert seen.all(), "an item is on no list"
        # lists of another shape in place of this one's: the kernel falls back to its fixed order
        other = cache._wgrad_item_lists(block_rows + 1024, tile[0], tile[1], ci, co)
        if other is not None and int(other.cpu().numpy()[1]) != items:
            setattr(cache, f"_wgrad_lists_{block_rows}_{tile[0]}_{tile[1]}_{ci}_{co}", other)
            with _force_schedule(wgrad=True, tile_rows=tile[0], tile_cols=tile[1], block_rows=block_rows, stream=1):
                gw, gb = impl._wgrad(g.to(gpu_device), f.to(gpu_device), cache, 27, with_bias=True, bias_offset=13)
            assert torch.equal(gw.cpu(), outs[False][0])
    finally:
        impl.WGRAD_BALANCED_LISTS = old
    assert torch.equal(outs[True][0], outs[False][0]) and torch.equal(outs[True][1], outs[False][1])
    # beyond 4 096 items or 12 voxel blocks and below 2 048 voxels the library makes no lists
    L = nat.lib()
    assert L.fgx_wgrad_item_lists_count(nat.sz(2047), C.c_int(27), C.c_int(256), C.c_int(256), C.c_int(128), C.c_int(128), C.c_int(1024)) == 0
    assert L.fgx_wgrad_item_lists_count(nat.sz(13 * 1024), C.c_int(27), C.c_int(32), C.c_int(32), C.c_int(32), C.c_int(32), C.c_int(1024)) == 0
    assert L.fgx_wgrad_item_lists_count(nat.sz(12 * 1024), C.c_int(27), C.c_int(32), C.c_int(32), C.c_int(32), C.c_int(32), C.c_int(1024)) == 4 + 256 + 27 * 12
    assert L.fgx_wgrad_item_lists_count(nat.sz(2048), C.c_int(27), C.c_int(256), C.c_int(256), C.c_int(128), C.c_int(128), C.c_int(1024)) == 4 + 256 + 27 * 4 * 2
    assert L.fgx_wgrad_item_lists_count(nat.sz(1 << 20), C.c_int(27), C.c_int(256), C.c_int(256), C.c_int(128), C.c_int(128), C.c_int(4096)) == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("res,ci,co,tile,sub_rows,lead,max_polls", [
    (32, 128, 128, 128, 256, 3, 2000), (48, 128, 128, 128, 128, 1, 2000), (24, 64, 64, 64, 64, 3, 2000),
    (32, 96, 40, 128, 512, 0, 3), (40, 48, 64, 64, 100000, 3, 2000), (64, 128, 128, 128, 1024, 2, 0),
    (16, 128, 64, 128, 64, 3, 2000)])
def test_sweep_wgrad_matches_oracle(gpu_device, dtype, res, ci, co, tile, sub_rows, lead, max_polls):
    """wgrad as the paced sweep, forced on small shells: sub-blocks far smaller than in production (most parts a step or
    two long, ragged steps everywhere), one sub-block for everything, channel counts below the tile, pacing with no
    lead and a poll limit that runs out (the workgroups then go on unpaced), and pacing switched off."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    _say(f"sweep wgrad res={res} ci={ci} co={co} tile={tile} sub_rows={sub_rows} lead={lead} polls={max_polls} {dtype}")
    coords_np = reference_test_shell(res)
    shape = torch.Size([1, ci, res, res, res])
    old = impl.WGRAD_SWEEP_LEAD, impl.WGRAD_SWEEP_MAX_POLLS
    impl.WGRAD_SWEEP_LEAD, impl.WGRAD_SWEEP_MAX_POLLS = lead, max_polls
    try:
        with _force_schedule(wgrad=True, tile_rows=tile, tile_cols=tile, block_rows=sub_rows, stream=2):
            cache, _ = _run_and_check(coords_np, shape, ci, co, dtype, gpu_device, seed=31)
        assert any(k.startswith("_wgrad_sweep_plan_") for k in vars(cache))
    finally:
        impl.WGRAD_SWEEP_LEAD, impl.WGRAD_SWEEP_MAX_POLLS = old


def test_sweep_wgrad_is_reproducible_and_close_to_the_block_major_kernel(gpu_device):
    """Two runs of the sweep give the same bits (fixed summation order); against the block-major streaming kernel the
    difference is fp32 rounding of a different order of additions."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    _say("sweep wgrad vs streaming wgrad")
    res, c = 64, 128
    coords_np = reference_test_shell(res)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([1, c, res, res, res])
    f, _, _, g = _case(coords_np, c, c, torch.float16, 35)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    outs = []
    for stream, rows in ((2, 512), (2, 512), (1, 4096)):
        with _force_schedule(wgrad=True, tile_rows=128, tile_cols=128, block_rows=rows, stream=stream):
            gw, gb = impl._wgrad(g.to(gpu_device), f.to(gpu_device), cache, 27, with_bias=True, bias_offset=13)
            outs.append((gw.cpu(), gb.cpu()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    assert eg.max_rel_err(outs[0][0], outs[2][0].double()) <= 2e-3
    assert eg.max_rel_err(outs[0][1], outs[2][1].double()) <= 2e-3


def test_sweep_wgrad_give_up_word_turns_the_result_into_nan(gpu_device):
    """A sweep wavefront whose wait for data runs out of looks goes on and sets its give-up word; the reduction then
    writes NaN everywhere.  Checked on the reduction alone: a normal sweep fills the scratch (all give-up words 0, result
    as usual), then one word is set by hand and only the reduction is run again -- no kernel is made to wait."""
    import ctypes as C
    from flexgemm_amd import _native as nat
    _say("sweep wgrad: give-up word -> NaN")
    L = nat.lib()
    res, ci, co, v, sub_rows, tile = 32, 128, 64, 27, 256, 128
    dtype = torch.float16
    code = nat.DTYPE_CODE[dtype]
    coords_np = reference_test_shell(res)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([1, ci, res, res, res])
    f, _, _, g = _case(coords_np, ci, co, dtype, 37)
    f, g = f.to(gpu_device), g.to(gpu_device)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    cache._ensure_pairs()
    seg_host = cache._seg_host()
    n = f.shape[0]
    plan = cache._wgrad_sweep_plan(sub_rows)
    seg_arr = (C.c_uint32 * (v + 1))(*seg_host)
    with torch.cuda.device(gpu_device):
        scratch = nat.workspace(L.fgx_wgrad_sweep_scratch_bytes(C.c_int(ci), C.c_int(co)), gpu_device)
        scratch.fill_(0xFF)                          # stale give-up words from "an earlier call": the sweep overwrites them
        offset = C.c_size_t(0)
        words = L.fgx_wgrad_sweep_giveup_words(C.c_int(ci), C.c_int(co), C.byref(offset))
        assert words > 0 and offset.value % 256 == 0 and offset.value + words * 4 <= scratch.numel()
        flags = scratch[offset.value:offset.value + words * 4].view(torch.int32)
        gw = torch.empty((co, v, ci), dtype=dtype, device=gpu_device)
        gb = torch.empty((co,), dtype=dtype, device=gpu_device)
        nat.check(L.fgx_conv_wgrad_sweep(
            C.c_int(code), nat.ptr(g), nat.ptr(f), nat.ptr(cache["valid_signal_i"]), nat.ptr(cache["valid_signal_o"]),
            seg_arr, nat.ptr(plan), nat.sz(n), nat.sz(n), C.c_int(ci), C.c_int(co), C.c_int(v), C.c_int(tile),
            C.c_int(sub_rows), C.c_int(3), C.c_int(0), nat.ptr(scratch), nat.ptr(gw), nat.ptr(gb), C.c_int(13), nat.stream()))
        torch.cuda.synchronize()
        assert int(flags.abs().max()) == 0, "a sweep wavefront gave up waiting on a healthy run"
        assert bool(torch.isfinite(gw.float()).all()) and bool(torch.isfinite(gb.float()).all())

        def reduce_again():
            gw2 = torch.zeros_like(gw)
            gb2 = torch.zeros_like(gb)
            nat.check(L.fgx_wgrad_sweep_reduce(
                C.c_int(code), nat.ptr(plan), nat.sz(n), nat.sz(seg_host[-1]), C.c_int(ci), C.c_int(co), C.c_int(v),
                C.c_int(sub_rows), nat.ptr(scratch), nat.ptr(gw2), nat.ptr(gb2), C.c_int(13), nat.stream()))
            torch.cuda.synchronize()
            return gw2, gb2

        gw2, gb2 = reduce_again()                    # untouched scratch: the reduction alone gives the same bits
        assert torch.equal(gw2, gw) and torch.equal(gb2, gb)
        for word in (0, words // 2 + 3, words - 1):  # any wavefront's word poisons everything
            flags.zero_()
            flags[word] = 1
            gw2, gb2 = reduce_again()
            assert bool(torch.isnan(gw2.float()).all()), f"give-up word {word} set, grad_weight not all NaN"
            assert bool(torch.isnan(gb2.float()).all()), f"give-up word {word} set, grad_bias not all NaN"
        flags.zero_()
        gw2, gb2 = reduce_again()
        assert torch.equal(gw2, gw) and torch.equal(gb2, gb)


def test_streaming_wgrad_equals_tiled_wgrad_bitwise(gpu_device):
    """Same 16-pair MFMA blocks in the same order inside every (voxel block, offset) item, same block-ordered
    reduction: the two wgrad kernels agree bit for bit."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    _say("stream wgrad vs tiled wgrad, bitwise")
    res, c = 40, 128
    coords_np = reference_test_shell(res)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    shape = torch.Size([1, c, res, res, res])
    f, _, _, g = _case(coords_np, c, c, torch.float16, 33)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    outs = []
    for stream in (0, 1):
        with _force_schedule(wgrad=True, tile_rows=128, tile_cols=128, block_rows=1024, stream=stream):
            outs.append(impl._wgrad(g.to(gpu_device), f.to(gpu_device), cache, 27).cpu())
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("name,res,c", [("cfg2", 64, 256), ("cfg3", 128, 128), ("cfg4", 128, 32), ("cfg5", 32, 1024)])
def test_scaled_down_benchmark_configs(gpu_device, name, res, c):
    """The benchmark configurations at a resolution the float64 oracle finishes in seconds."""
    _say(f"conv {name} at res {res}")
    wl = make_workload(name, res=res, with_values=False)
    _run_and_check(wl.coords.numpy(), wl.shape, c, c, wl.dtype, gpu_device, seed=11)


def test_cfg5_fp32_variant(gpu_device):
    _say("conv cfg5 fp32 variant at res 32")
    wl = make_workload("cfg5", res=32, with_values=False)
    _, errs = _run_and_check(wl.coords.numpy(), wl.shape, 1024, 1024, torch.float32, gpu_device, seed=12)
    assert max(e[1] for e in errs) <= 1e-4


WGRAD_OFFSETS = (0, 4, 13, 22, 26, 17)


def _full_size_check(wl, dt, sample, dev, seed):
    """A benchmark configuration at full size through the public operator: a random sample of output rows against the
    float64 oracle (forward and input gradient); the weight gradient of six offsets (the corners 0 and 26, the face
    neighbors 4 and 22, the centre 13 and offset 17), every element of their [Co, Ci] slices, against the float64
    oracle; the inner-product identities <conv(f), g> = <f, dgrad(g)> = <W, wgrad> over the whole tensors; and the
    bias gradient against the column sums."""
    c = wl.feats.shape[1]
    f = wl.feats.to(dt).to(dev).requires_grad_(True)
    w = wl.weight.to(dt).to(dev).requires_grad_(True)
    b = wl.bias.to(dt).to(dev).requires_grad_(True)
    g = wl.grad.to(dt)
    coords = wl.coords.to(dev)
    out, cache = sparse_submanifold_conv3d(f, coords, wl.shape, w, b)
    out.backward(g.to(dev))
    torch.cuda.synchronize()
    nmap = cache.neighbor_map.cpu().view(torch.int32)
    rows = torch.randperm(wl.n, generator=torch.Generator().manual_seed(seed))[:sample]
    f64, w64, b64, g64 = f.detach().cpu().double(), w.detach().cpu().double(), b.detach().cpu().double(), g.double()
    ref_rows = eg.forward(f64, nmap[rows], w64, b64)
    _assert_close(out[rows.to(dev)], ref_rows, dt, "forward sample")
    ref_gi = torch.mm(eg._im2col(g64, torch.flip(nmap[rows].long(), [1])), w64.reshape(c, 27, c).transpose(0, 1).reshape(27 * c, c))
    _assert_close(f.grad[rows.to(dev)], ref_gi, dt, "dgrad sample")
    gw = w.grad.detach().cpu().reshape(c, 27, c)
    for v in WGRAD_OFFSETS:
        _say(f"  wgrad slice of offset {v}")
        _assert_close(gw[:, v], eg.weight_grad_offset(g64, f64, nmap, v), dt, f"wgrad offset {v}")
    # inner-product identities in float64 from the GPU results (bias-free part)
    conv_nobias = out.detach().cpu().double() - b64
    lhs = (conv_nobias * g64).sum()
    mid = (f64 * f.grad.cpu().double()).sum()
    rhs = (w64 * w.grad.cpu().double()).sum()
    scale = float((conv_nobias.abs() * g64.abs()).sum())
    assert abs(lhs - mid) / scale < 1e-3 and abs(lhs - rhs) / scale < 1e-3
    _assert_close(b.grad, g64.sum(0), dt, "dbias")
    return cache


@pytest.mark.parametrize("name,sample", [("cfg3", 4096), ("cfg2", 2048), ("cfg4", 4096), ("cfg5", 512)])
def test_full_size_properties(gpu_device, name, sample):
    """Configurations 2, 3, 4 and 5 at full size, in their own dtypes (cfg3: 669 288 voxels, C = 128, fp16)."""
    wl = make_workload(name)
    _say(f"conv {name} full size, n={wl.n} C={wl.feats.shape[1]} {wl.dtype}")
    _full_size_check(wl, wl.dtype, sample, gpu_device, seed=1)


def test_full_size_cfg4_through_the_resident_row_kernels(gpu_device):
    """Configuration 4 at full size (2.67 million voxels, C = 32, bf16) with the resident-row kernels forced on: the
    automatic policy would send a cache's first products to the streaming kernels, which the test above covers."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    wl = make_workload("cfg4")
    _say(f"conv cfg4 full size through the resident-row kernels, n={wl.n}")
    old = impl.spconv.NARROW_RESIDENT
    impl.spconv.NARROW_RESIDENT = "on"
    try:
        cache = _full_size_check(wl, wl.dtype, 4096, gpu_device, seed=3)
    finally:
        impl.spconv.NARROW_RESIDENT = old
    assert hasattr(cache, "_narrow_plan_buf") and getattr(cache, "_narrow_overflows", None) == 0, \
        "the resident-row kernels did not run"


@pytest.mark.parametrize("c", [16, 128])
def test_more_than_2_to_the_24_voxels_and_operands_past_4_gib(gpu_device, c):
    """A dense block of 257 x 256 x 256 = 16 842 752 voxels, past the 24-bit row numbers of the weight-gradient sweep; with
    C = 128 in fp16 every operand is 4.3 GB, past the 32-bit byte offsets of the streaming kernels, so the products take
    the kernels with 64-bit addressing.  In a dense block the neighbor of a voxel is a fixed step in its row number (the
    27 steps are read off the oracle's map of a small block), which gives, without the oracle's loops: the map of sampled
    rows and of the rows around 2^24, bit for bit; the pair count in closed form; forward and input gradient of the
    sampled rows, every element of the weight gradient of six offsets (slices of the block against each other) and the
    bias gradient, all in float64 torch arithmetic, to 1e-2 of the largest value."""
    dev = gpu_device
    X, Y, Z = 257, 256, 256
    n = X * Y * Z
    _say(f"dense block of {n} voxels, C={c}")
    sx, sy, sz = 5, 4, 4
    small = np.stack([np.zeros(sx * sy * sz, np.int32)] + [a.reshape(-1).astype(np.int32) for a in
                                                         np.meshgrid(np.arange(sx), np.arange(sy), np.arange(sz), indexing="ij")], 1)
    smap = nb.neighbor_map(small, (1, 1, sx, sy, sz), (3, 3, 3), (1, 1, 1)).view(np.int32)
    centre = (2 * sy + 1) * sz + 1
    assert (smap[centre] >= 0).all()
    delta = small[smap[centre]][:, 1:] - small[centre][1:]              # [27, 3]: the step of every kernel offset
    delta_t = torch.from_numpy(delta).to(dev).long()
    coords = torch.stack([torch.zeros(n, dtype=torch.int32, device=dev),
                          torch.arange(X, device=dev, dtype=torch.int32).repeat_interleave(Y * Z),
                          torch.arange(Y, device=dev, dtype=torch.int32).repeat_interleave(Z).repeat(X),
                          torch.arange(Z, device=dev, dtype=torch.int32).repeat(X * Y)], 1).contiguous()

    def neighbors(rows):                # [S] -> [S, 27] row numbers, -1 outside the block
        x, y, z = rows // (Y * Z), (rows // Z) % Y, rows % Z
        nx, ny, nz = x[:, None] + delta_t[:, 0], y[:, None] + delta_t[:, 1], z[:, None] + delta_t[:, 2]
        inside = (nx >= 0) & (nx < X) & (ny >= 0) & (ny < Y) & (nz >= 0) & (nz < Z)
        return torch.where(inside, (nx * Y + ny) * Z + nz, torch.full_like(nx, -1))

    def rel(got, ref):
        return float((got.double() - ref).abs().max() / ref.abs().max())

    dt = torch.float16
    shape = torch.Size([1, c, X, Y, Z])
    g = torch.Generator(device=dev).manual_seed(c)
    f = torch.randn(n, c, generator=g, device=dev, dtype=dt).requires_grad_(True)
    w = (torch.randn(c, 3, 3, 3, c, generator=g, device=dev) / (27 * c) ** 0.5).to(dt).requires_grad_(True)
    b = torch.randn(c, generator=g, device=dev).to(dt).requires_grad_(True)
    go = torch.randn(n, c, generator=g, device=dev, dtype=dt)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    rows = torch.cat([torch.randint(0, n, (4096,), device=dev, generator=g),
                      torch.tensor([0, n - 1, (1 << 24) - 1, 1 << 24, (1 << 24) + 1], device=dev)])
    nbr = neighbors(rows)
    assert torch.equal(cache.neighbor_map.view(torch.int32)[rows].long(), nbr), "neighbor map"
    assert int(cache._seg_host()[-1]) == sum((X - abs(int(d[0]))) * (Y - abs(int(d[1]))) * (Z - abs(int(d[2]))) for d in delta)
    _say("  forward and backward")
    out = sparse_submanifold_conv3d(f, coords, shape, w, b, cache)[0]
    out.backward(go)
    torch.cuda.synchronize()
    w64 = w.detach().double().reshape(c, 27, c)
    fg = f.detach()[nbr.clamp(min=0)].double() * (nbr >= 0)[:, :, None]
    assert rel(out.detach()[rows], torch.einsum("svc,ovc->so", fg, w64) + b.detach().double()) < 1e-2, "forward"
    back = torch.flip(nbr, [1])         # the voxel that has this one as its neighbor at offset v is the neighbor at V - 1 - v
    gg = go[back.clamp(min=0)].double() * (back >= 0)[:, :, None]
    assert rel(f.grad[rows], torch.einsum("svo,ovc->sc", gg, w64)) < 1e-2, "input gradient"
    gw = w.grad.reshape(c, 27, c)
    F, G = f.detach().view(X, Y, Z, c), go.view(X, Y, Z, c)
    for v in WGRAD_OFFSETS:
        _say(f"  wgrad slice of offset {v}")
        dx, dy, dz = (int(t) for t in delta[v])
        ref = torch.zeros(c, c, dtype=torch.float64, device=dev)
        x_end = min(X, X - dx)
        for x0 in range(max(0, -dx), x_end, 16):
            x1 = min(x0 + 16, x_end)
            gs = G[x0:x1, max(0, -dy):min(Y, Y - dy), max(0, -dz):min(Z, Z - dz)].reshape(-1, c).double()
            fs = F[x0 + dx:x1 + dx, max(0, dy):min(Y, Y + dy), max(0, dz):min(Z, Z + dz)].reshape(-1, c).double()
            ref += gs.t() @ fs
        assert rel(gw[:, v], ref) < 1e-2, f"weight gradient of offset {v}"
    ref = torch.zeros(c, dtype=torch.float64, device=dev)
    for x0 in range(0, X, 16):
        ref += G[x0:x0 + 16].reshape(-1, c).double().sum(0)
    assert rel(b.grad, ref) < 1e-2, "bias gradient"
    del f, w, b, go, out, cache, fg, gg, F, G
    torch.cuda.empty_cache()


def test_full_size_cfg5_fp32_variant(gpu_device):
    """Configuration 5's fp32-input variant (fp32 accumulation) at full size: 42 608 voxels, C = 1024, tolerance 1e-4."""
    wl = make_workload("cfg5")
    _say(f"conv cfg5 fp32 variant full size, n={wl.n}")
    _full_size_check(wl, torch.float32, 256, gpu_device, seed=2)


def test_cfg1_whole_tensors(gpu_device):
    """Configuration 1 (res-64 shell, 10 208 voxels, Ci = Co = 64, fp32) on the HIP path: forward with the workload's
    own values against the float64 oracle over the whole tensor, and the backward pass as well."""
    wl = make_workload("cfg1")
    _say(f"conv cfg1, n={wl.n}")
    assert wl.n == 10208 and wl.dtype == torch.float32
    dev = gpu_device
    f = wl.feats.to(dev).requires_grad_(True)
    w = wl.weight.to(dev).requires_grad_(True)
    b = wl.bias.to(dev).requires_grad_(True)
    out, cache = sparse_submanifold_conv3d(f, wl.coords.to(dev), wl.shape, w, b)
    out.backward(wl.grad.to(dev))
    torch.cuda.synchronize()
    nmap = torch.from_numpy(nb.neighbor_map(wl.coords.numpy(), tuple(wl.shape)).view(np.int32))
    assert torch.equal(cache.neighbor_map.cpu().view(torch.int32), nmap)
    f64, w64, b64, g64 = wl.feats.double(), wl.weight.double(), wl.bias.double(), wl.grad.double()
    _assert_close(out, eg.forward(f64, nmap, w64, b64), torch.float32, "forward")
    ref_gi, ref_gw, ref_gb = eg.backward(g64, f64, nmap, w64)
    _assert_close(f.grad, ref_gi, torch.float32, "dgrad")
    _assert_close(w.grad, ref_gw, torch.float32, "wgrad")
    _assert_close(b.grad, ref_gb, torch.float32, "dbias")


def test_very_wide_output_runs_the_tiled_kernel(gpu_device):
    """2048 output columns: the persistent kernel's staged bias no longer fits a CU's LDS, the table leaves the layer
    to the tiled kernel (forward: Co columns; dgrad: Ci columns)."""
    res = 20
    coords_np = reference_test_shell(res)
    _say(f"conv Co=2048 / Ci=2048, n={len(coords_np)}")
    _run_and_check(coords_np, torch.Size([1, 64, res, res, res]), 64, 2048, torch.float16, gpu_device, seed=3)
    _run_and_check(coords_np, torch.Size([1, 2048, res, res, res]), 2048, 64, torch.float16, gpu_device, seed=4)


def test_wide_channels_with_a_32x32_streaming_wgrad_tile_fall_back(gpu_device):
    """A caller that asks for the 32 x 32 streaming wgrad tile with more than 32 channels on both sides gets the tiled
    kernel: the scratch size the library quotes has no room for that tile's four partial products per block there."""
    res, c = 24, 64
    coords_np = reference_test_shell(res)
    _say(f"wgrad tile 32 stream=1 at C={c}")
    with _force_schedule(wgrad=True, tile_rows=32, tile_cols=32, block_rows=512, stream=1):
        _run_and_check(coords_np, torch.Size([1, c, res, res, res]), c, c, torch.float16, gpu_device, seed=29)


def test_weight_panel_cache_keeps_results_and_follows_weight_updates(gpu_device):
    """Opt-in reuse of the repacked weight panels: same bits as without it, a panel kept from the second call on, an
    in-place weight update seen through the version counter, the byte budget respected, bytes released with the weight."""
    import gc
    from flexgemm_amd.ops import spconv as cfg
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    res, c = 32, 64
    coords_np = reference_test_shell(res)
    shape = torch.Size([1, c, res, res, res])
    feats, weight, bias, grad = _case(coords_np, c, c, torch.float16, seed=11)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)

    def step(w, b):
        f = feats.to(gpu_device).requires_grad_(True)
        w.grad = None
        out, _ = sparse_submanifold_conv3d(f, coords, shape, w, b, neighbor_cache=cache)
        out.backward(grad.to(gpu_device))
        return out.detach().clone(), f.grad.clone(), w.grad.clone()

    w = weight.to(gpu_device).requires_grad_(True)
    b = bias.to(gpu_device)
    plain = step(w, b)
    kept_before = impl._panel_bytes_kept
    cfg.set_weight_panel_cache(True)
    try:
        _say("panel cache: three steps with one weight")
        for i in range(3):
            got = step(w, b)
            assert all(torch.equal(x, y) for x, y in zip(got, plain)), f"step {i} differs from the uncached result"
            panels = [e for e in w._fgx_weight_panels.values() if e[1] is not None]
            assert len(panels) == (0 if i == 0 else 2), f"step {i}: {len(panels)} panels kept"      # forward and dgrad
        assert impl._panel_bytes_kept > kept_before
        _say("panel cache: in-place update")
        with torch.no_grad():
            w.mul_(0.5)
        got = step(w, b)
        cfg.set_weight_panel_cache(False)
        want = step(w, b)
        cfg.set_weight_panel_cache(True)
        assert all(torch.equal(x, y) for x, y in zip(got, want))
        assert not torch.equal(got[0], plain[0])
        assert all(e[1] is None for e in w._fgx_weight_panels.values())       # the stale panels are gone
        _say("panel cache: zero budget keeps nothing")
        cfg.set_weight_panel_cache(True, max_bytes=0)
        w2 = weight.to(gpu_device).requires_grad_(True)
        for _ in range(3):
            got = step(w2, b)
        assert all(torch.equal(x, y) for x, y in zip(got, plain))
        assert all(e[1] is None for e in w2._fgx_weight_panels.values())
        del w, w2, got, want, panels
        gc.collect()
        assert impl._panel_bytes_kept == kept_before
    finally:
        cfg.set_weight_panel_cache(False, max_bytes=4 << 30)


@pytest.mark.parametrize("res,c", [(24, 64), (64, 128), (16, 1024)])
def test_forward_replays_from_a_hip_graph(gpu_device, res, c):
    """Two stacked layers captured into a HIP graph (the library calls no allocation, memset, copy or synchronisation,
    so a warmed-up forward records kernels only): every replay, with new input values and eager work of the same
    operator between the replays, equals the eager result bit for bit.  Sizes cover the tiled kernel with split-K, the
    streaming kernel and the wide-channel case."""
    coords_np = reference_test_shell(res)
    shape = torch.Size([1, c, res, res, res])
    coords = torch.from_numpy(coords_np).to(gpu_device)
    n = len(coords_np)
    g = torch.Generator().manual_seed(res * c)
    ws = [(torch.randn(c, 3, 3, 3, c, generator=g) / math.sqrt(27 * c)).half().to(gpu_device) for _ in range(2)]
    bs = [torch.randn(c, generator=g).half().to(gpu_device) for _ in range(2)]
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), False)

    def stack(x):
        for w, b in zip(ws, bs):
            x = sparse_submanifold_conv3d(x, coords, shape, w, b, cache)[0]
        return x

    static_in = torch.randn(n, c, generator=g).half().to(gpu_device)
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                stack(static_in)                 # builds the plans and the schedule lookups the capture must not build
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        _say(f"graph capture res={res} c={c}")
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_out = stack(static_in)
        for k in range(4):
            x = torch.randn(n, c, generator=g).half().to(gpu_device)
            static_in.copy_(x)
            graph.replay()
            eager = stack(x)                     # the program's own eager work between the replays
            torch.cuda.synchronize()
            assert torch.equal(static_out, eager), f"replay {k} differs from the eager result"


def test_graph_captured_with_the_panel_cache_on_follows_weight_updates(gpu_device):
    """With the weight panel cache on and panels already kept, a captured forward still packs its panels inside the
    graph: after an in-place weight update every replay equals the eager result of the updated weights."""
    from flexgemm_amd.ops import spconv as cfg
    res, c = 24, 64
    coords_np = reference_test_shell(res)
    shape = torch.Size([1, c, res, res, res])
    coords = torch.from_numpy(coords_np).to(gpu_device)
    n = len(coords_np)
    g = torch.Generator().manual_seed(77)
    w = (torch.randn(c, 3, 3, 3, c, generator=g) / math.sqrt(27 * c)).half().to(gpu_device)
    b = torch.randn(c, generator=g).half().to(gpu_device)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), False)
    static_in = torch.randn(n, c, generator=g).half().to(gpu_device)
    cfg.set_weight_panel_cache(True)
    try:
        with torch.no_grad():
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for _ in range(3):          # the second and third call keep and reuse a panel
                    sparse_submanifold_conv3d(static_in, coords, shape, w, b, cache)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            assert any(e[1] is not None for e in w.__dict__["_fgx_weight_panels"].values())
            _say("graph capture with kept weight panels")
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                static_out = sparse_submanifold_conv3d(static_in, coords, shape, w, b, cache)[0]
            for k in range(3):
                w.mul_(-0.5).add_(0.01)     # an optimizer step's in-place update
                graph.replay()
                eager = sparse_submanifold_conv3d(static_in, coords, shape, w, b, cache)[0]
                torch.cuda.synchronize()
                assert torch.equal(static_out, eager), f"replay {k} used stale weights"
    finally:
        cfg.set_weight_panel_cache(False)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("res,ci,co", [(48, 128, 128), (24, 64, 96), (8, 256, 64), (16, 20, 12)])
def test_relu_in_the_epilogue_equals_relu_after_the_operator(gpu_device, dtype, res, ci, co):
    """sparse_submanifold_conv3d_relu against torch.relu(sparse_submanifold_conv3d): rounding is monotonic and keeps
    the sign, so the fused output equals the composed one bit for bit, and so do all gradients (the mask is the same).
    Shapes cover the streaming kernel, the tiled kernel, its split-K reduction and zero-padded channel counts; one
    comparison against the float64 oracle guards the pair against a common mistake."""
    from flex_gemm.ops.spconv import sparse_submanifold_conv3d_relu
    coords_np = reference_test_shell(res)
    shape = torch.Size([1, ci, res, res, res])
    feats, weight, bias, grad = _case(coords_np, ci, co, dtype, seed=res + ci)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    results = []
    for fused in (False, True):
        f = feats.to(gpu_device).requires_grad_(True)
        w = weight.to(gpu_device).requires_grad_(True)
        b = bias.to(gpu_device).requires_grad_(True)
        if fused:
            out, _ = sparse_submanifold_conv3d_relu(f, coords, shape, w, b, neighbor_cache=cache)
        else:
            out = torch.relu(sparse_submanifold_conv3d(f, coords, shape, w, b, neighbor_cache=cache)[0])
        out.backward(grad.to(gpu_device))
        torch.cuda.synchronize()
        results.append((out.detach(), f.grad, w.grad, b.grad))
    _say(f"fused relu res={res} ci={ci} co={co} {dtype}")
    for name, a, b_ in zip(("output", "dgrad", "wgrad", "dbias"), results[0], results[1]):
        assert torch.equal(a, b_), f"{name}: fused and composed results differ"
    assert (results[1][0] >= 0).all() and (results[1][0] == 0).any() and (results[1][0] > 0).any()
    nmap = torch.from_numpy(nb.neighbor_map(coords_np, tuple(shape), (3, 3, 3), (1, 1, 1)).view(np.int32))
    ref = torch.relu(eg.forward(feats.double(), nmap, weight.double(), bias.double()))
    _assert_close(results[1][0], ref, dtype, "fused relu forward")
    # without a bias, and without gradients
    with torch.no_grad():
        a = sparse_submanifold_conv3d_relu(feats.to(gpu_device), coords, shape, weight.to(gpu_device), None, cache)[0]
        b_ = torch.relu(sparse_submanifold_conv3d(feats.to(gpu_device), coords, shape, weight.to(gpu_device), None, cache)[0])
    assert torch.equal(a, b_)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("res,ci,co", [(48, 128, 128), (24, 64, 96), (8, 256, 64), (40, 32, 32)])
def test_relu_bit_mask_of_the_epilogue_and_its_use_in_backward(gpu_device, dtype, res, ci, co):
    """The fused-ReLU forward also writes one bit per output, "greater than zero" (streaming kernel, tiled kernel, split-K
    reduction); backward masks the gradient with those bits in one pass.  The bits must equal (output > 0) exactly, and
    fgx_relu_mask_apply must equal torch.where on gradients that hold NaN, infinities and negative zero."""
    import ctypes as C
    from flexgemm_amd import _native as nat
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    _say(f"relu bit mask res={res} ci={ci} co={co} {dtype}")
    coords_np = reference_test_shell(res)
    shape = torch.Size([1, ci, res, res, res])
    feats, weight, bias, grad = _case(coords_np, ci, co, dtype, seed=res + co)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    masks = []
    out = SubMConv3dFunction._sparse_submanifold_conv_forward(feats.to(gpu_device), cache, weight.to(gpu_device),
                                                              bias.to(gpu_device), relu=True, relu_mask_out=masks)
    torch.cuda.synchronize()
    assert len(masks) == 1 and masks[0].dtype == torch.uint8 and masks[0].numel() == out.numel() // 8
    want = np.packbits((out.float().cpu().numpy() > 0).reshape(-1), bitorder="little")
    assert np.array_equal(masks[0].cpu().numpy(), want), "mask bits differ from (output > 0)"
    assert 0 < int(want.sum()) and (want != 0xFF).any()
    g = grad.to(gpu_device).clone()
    flat = g.view(-1)
    flat[0], flat[1], flat[2], flat[3] = float("nan"), float("inf"), float("-inf"), -0.0
    flat[-1] = float("nan")
    got = impl._relu_mask_apply(g, masks[0])
    torch.cuda.synchronize()
    ref = torch.where(out > 0, g, torch.zeros((), dtype=dtype, device=gpu_device))
    assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), "masked gradient differs from torch.where"
    # in place, as the header allows
    nat.check(nat.lib().fgx_relu_mask_apply(C.c_int(nat.DTYPE_CODE[dtype]), nat.ptr(g), nat.ptr(masks[0]), nat.sz(g.numel()),
                                            nat.ptr(g), nat.stream()))
    torch.cuda.synchronize()
    assert torch.equal(g.view(torch.int16), ref.view(torch.int16))
    # what the kernels refuse
    with pytest.raises(ValueError):
        nat.check(nat.lib().fgx_relu_mask_apply(C.c_int(nat.FGX_F32), nat.ptr(g), nat.ptr(masks[0]), nat.sz(g.numel()),
                                                nat.ptr(g), nat.stream()))
    with pytest.raises(ValueError):
        nat.check(nat.lib().fgx_relu_mask_apply(C.c_int(nat.DTYPE_CODE[dtype]), nat.ptr(g), nat.ptr(masks[0]), nat.sz(12),
                                                nat.ptr(g), nat.stream()))


@pytest.mark.parametrize("c,narrow", [(128, "auto"), (32, "on")])
def test_training_step_replays_from_a_hip_graph(gpu_device, c, narrow):
    """Forward and backward of two stacked layers captured once (whole-step capture: static input, gradients allocated
    by the captured backward) and replayed with new inputs; every replay equals the eager step bit for bit, with eager
    steps of the same layers running between the replays.  With 32 channels and the resident-row kernels forced on, the
    warm-up steps make the plan and read its header; the capture then records those kernels and nothing else."""
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    old_narrow = impl.spconv.NARROW_RESIDENT
    impl.spconv.NARROW_RESIDENT = narrow
    try:
        _graph_training_step(gpu_device, c, narrow == "on")
    finally:
        impl.spconv.NARROW_RESIDENT = old_narrow


def _graph_training_step(gpu_device, c, expect_narrow):
    res = 48
    coords_np = reference_test_shell(res)
    shape = torch.Size([1, c, res, res, res])
    coords = torch.from_numpy(coords_np).to(gpu_device)
    n = len(coords_np)
    g = torch.Generator().manual_seed(5)
    ws = [torch.nn.Parameter((torch.randn(c, 3, 3, 3, c, generator=g) / math.sqrt(27 * c)).half().to(gpu_device)) for _ in range(2)]
    bs = [torch.nn.Parameter(torch.randn(c, generator=g).half().to(gpu_device)) for _ in range(2)]
    params = ws + bs
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    upstream = torch.randn(n, c, generator=g).half().to(gpu_device)

    def step(x):
        h = x
        for w, b in zip(ws, bs):
            h = sparse_submanifold_conv3d(h, coords, shape, w, b, cache)[0]
        h.backward(upstream)
        return h

    static_in = torch.randn(n, c, generator=g).half().to(gpu_device)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            for p in params:
                p.grad = None
            step(static_in)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for p in params:
        p.grad = None                      # the captured backward allocates the gradients in the graph's pool
    _say("graph capture of a training step")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = step(static_in)
    static_grads = [p.grad for p in params]
    assert all(sg is not None for sg in static_grads)
    for k in range(3):
        x = torch.randn(n, c, generator=g).half().to(gpu_device)
        static_in.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        got = [static_out.clone()] + [sg.clone() for sg in static_grads]
        for p in params:
            p.grad = None
        want_out = step(x)                 # eager step between the replays
        torch.cuda.synchronize()
        want = [want_out.detach()] + [p.grad for p in params]
        for i, (a, b_) in enumerate(zip(got, want)):
            assert torch.equal(a, b_), f"replay {k}, tensor {i} differs from the eager step"
        for p, sg in zip(params, static_grads):
            p.grad = sg                    # hand the static gradient tensors back for the next replay
    assert hasattr(cache, "_narrow_plan_buf") == expect_narrow and (getattr(cache, "_narrow_overflows", None) == 0) == expect_narrow
