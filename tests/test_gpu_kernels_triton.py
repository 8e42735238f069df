"""`flex_gemm.kernels.triton` under the reference's names (flex_gemm/kernels/triton/spconv/__init__.py:1-13): the
kernel-level calls the reference's operators make (ops/spconv/submanifold_conv3d.py:174-209, 262-313;
ops/spconv/sparse_conv3d.py:304-339, 391-445), handed plain tensors, against the explicit gather-GEMM oracle in float64.
Tolerance: max relative error <= 1e-2 for fp16 / bf16, <= 1e-4 for fp32."""
import math
import sys

import numpy as np
import pytest
import torch

import flex_gemm
from flex_gemm import kernels
from flex_gemm.ops.spconv import SparseConv3dFunction, SubMConv3dFunction
from flexgemm_amd.workloads import reference_test_shell
from oracle import explicit_gemm as eg
from oracle import neighbor as nb
from oracle import sparse_conv as sc

TOL = {torch.float16: 1e-2, torch.bfloat16: 1e-2, torch.float32: 1e-4}
NAMES = [
    "sparse_submanifold_conv_fwd_implicit_gemm", "sparse_submanifold_conv_bwd_implicit_gemm",
    "sparse_submanifold_conv_fwd_implicit_gemm_splitk", "sparse_submanifold_conv_bwd_implicit_gemm_splitk",
    "sparse_submanifold_conv_fwd_masked_implicit_gemm", "sparse_submanifold_conv_bwd_masked_implicit_gemm",
    "sparse_submanifold_conv_fwd_masked_implicit_gemm_splitk", "sparse_submanifold_conv_bwd_masked_implicit_gemm_splitk",
    "sparse_conv_fwd_implicit_gemm", "sparse_conv_bwd_implicit_gemm",
    "sparse_conv_fwd_implicit_gemm_splitk", "sparse_conv_bwd_implicit_gemm_splitk",
    "sparse_conv_fwd_masked_implicit_gemm", "sparse_conv_bwd_masked_implicit_gemm",
    "sparse_conv_fwd_masked_implicit_gemm_splitk", "sparse_conv_bwd_masked_implicit_gemm_splitk",
]


def _say(msg):
    print(f"[kernels.triton] {msg}", file=sys.stderr, flush=True)


def _close(got, ref64, dtype, what):
    got = got.detach().cpu()
    tol = TOL[dtype]
    rms = max(float(ref64.double().pow(2).mean().sqrt()), 1e-30)
    e_metric = eg.calc_err(got.double() / rms, ref64.double() / rms)[0]
    e_scaled = eg.max_rel_err(got, ref64)
    assert e_metric <= tol and e_scaled <= tol, f"{what}: min(abs,rel)={e_metric:.3e} scaled={e_scaled:.3e} tol={tol}"


def test_names_and_switches_are_there():
    for name in NAMES:
        assert callable(getattr(kernels.triton, name)), name
        assert getattr(kernels.triton.spconv, name) is getattr(kernels.triton, name)
    # the assignment the reference's benchmarks make (tests/submconv/train_benchmark.py:135)
    before = flex_gemm.kernels.triton.spconv.config.allow_tf32
    flex_gemm.kernels.triton.spconv.config.allow_tf32 = True
    assert kernels.triton.config.allow_tf32 is True
    flex_gemm.kernels.triton.spconv.config.allow_tf32 = before


def test_host_tensors_are_refused():
    x = torch.zeros(4, 8)
    w = torch.zeros(8, 27, 8)
    nmap = torch.zeros(4, 27, dtype=torch.int32).view(torch.uint32)
    with pytest.raises(NotImplementedError):
        kernels.triton.sparse_submanifold_conv_fwd_implicit_gemm(x, w, None, nmap)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("res,ci,co", [(24, 64, 64), (40, 128, 128), (16, 20, 12)])
def test_submanifold_kernel_calls(gpu_device, dtype, res, ci, co):
    dev = gpu_device
    coords_np = reference_test_shell(res)
    n, v = len(coords_np), 27
    shape = torch.Size([1, ci, res, res, res])
    g = torch.Generator().manual_seed(res + ci)
    feats = torch.randn(n, ci, generator=g).to(dtype)
    weight = (torch.randn(co, v, ci, generator=g) / math.sqrt(v * ci)).to(dtype)
    bias = torch.randn(co, generator=g).to(dtype)
    grad = torch.randn(n, co, generator=g).to(dtype)
    nmap_np = nb.neighbor_map(coords_np, tuple(shape), (3, 3, 3), (1, 1, 1))
    nmap_cpu = torch.from_numpy(nmap_np.view(np.int32))
    w5 = weight.double().reshape(co, 3, 3, 3, ci)
    ref_out = eg.forward(feats.double(), nmap_cpu, w5, bias.double())
    ref_gi, ref_gw, ref_gb = eg.backward(grad.double(), feats.double(), nmap_cpu, w5)
    ref_gw = ref_gw.reshape(co, v, ci)

    cache = SubMConv3dFunction._compute_neighbor_cache(torch.from_numpy(coords_np).to(dev), shape, (3, 3, 3), (1, 1, 1), True)
    f = feats.to(dev).requires_grad_(True)
    w = weight.to(dev).requires_grad_(True)
    b = bias.to(dev).requires_grad_(True)
    go = grad.to(dev)
    nmap = cache["neighbor_map"]

    for tag in ("", "_splitk"):
        _say(f"submanifold res={res} ci={ci} co={co} {dtype} non-masked{tag}")
        fwd = getattr(kernels.triton, "sparse_submanifold_conv_fwd_implicit_gemm" + tag)
        bwd = getattr(kernels.triton, "sparse_submanifold_conv_bwd_implicit_gemm" + tag)
        out = fwd(f, w, b, nmap)
        assert out.dtype == dtype and tuple(out.shape) == (n, co)
        _close(out, ref_out, dtype, "forward")
        gi, gw, gb = bwd(go, f, w, b, nmap)
        assert tuple(gw.shape) == (co, v, ci)
        _close(gi, ref_gi, dtype, "dgrad"), _close(gw, ref_gw, dtype, "wgrad"), _close(gb, ref_gb, dtype, "dbias")

        _say(f"submanifold res={res} ci={ci} co={co} {dtype} masked{tag}")
        fwd = getattr(kernels.triton, "sparse_submanifold_conv_fwd_masked_implicit_gemm" + tag)
        bwd = getattr(kernels.triton, "sparse_submanifold_conv_bwd_masked_implicit_gemm" + tag)
        out = fwd(f, w, b, nmap, cache["sorted_idx"], cache.valid_kernel_callback, cache.valid_kernel_seg_callback)
        _close(out, ref_out, dtype, "forward")
        gi, gw, gb = bwd(go, f, w, b, nmap, cache["sorted_idx"], cache["valid_kernel_callback"], cache["valid_kernel_seg_callback"],
                         cache["valid_signal_i"], cache["valid_signal_o"], cache["valid_signal_seg"])
        _close(gi, ref_gi, dtype, "dgrad"), _close(gw, ref_gw, dtype, "wgrad"), _close(gb, ref_gb, dtype, "dbias")
        # the same call again finds its tables on the map tensor and gives the same bits
        out2 = fwd(f, w, b, nmap, cache["sorted_idx"], cache.valid_kernel_callback, cache.valid_kernel_seg_callback)
        assert torch.equal(out2, out)

    # gradients only where asked for; no bias
    gi, gw, gb = kernels.triton.sparse_submanifold_conv_bwd_masked_implicit_gemm_splitk(
        go, f.detach(), w, None, nmap, cache["sorted_idx"], None, None, cache["valid_signal_i"], cache["valid_signal_o"],
        cache["valid_signal_seg"])
    assert gi is None and gb is None
    _close(gw, ref_gw, dtype, "wgrad alone")
    out = kernels.triton.sparse_submanifold_conv_fwd_masked_implicit_gemm_splitk(f, w, None, nmap, cache["sorted_idx"])
    _close(out, ref_out - bias.double(), dtype, "forward without bias")

    # any permutation serves as sorted_idx, and the pair lists may be left to the callee
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(1)).to(dev)
    out = kernels.triton.sparse_submanifold_conv_fwd_masked_implicit_gemm(f, w, b, nmap, perm)
    _close(out, ref_out, dtype, "forward, arbitrary order")
    gi, gw, gb = kernels.triton.sparse_submanifold_conv_bwd_masked_implicit_gemm(go, f, w, b, nmap, perm)
    _close(gi, ref_gi, dtype, "dgrad, arbitrary order"), _close(gw, ref_gw, dtype, "wgrad, derived pairs")
    assert len(nmap._fgx_kernel_tables) <= 4


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("geom", [((3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1)), ((2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1)),
                                  ((3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1))])
def test_generic_kernel_calls(gpu_device, dtype, geom):
    dev = gpu_device
    res, ci, co = 24, 64, 96
    ks, st, pd, dl = geom
    coords_np = reference_test_shell(res)
    shape = torch.Size([1, ci, res, res, res])
    oc_np = sc.output_coords(coords_np, tuple(shape), ks, st, pd, dl)
    m, l, v = len(coords_np), len(oc_np), ks[0] * ks[1] * ks[2]
    g = torch.Generator().manual_seed(v)
    feats = torch.randn(m, ci, generator=g).to(dtype)
    weight = (torch.randn(co, v, ci, generator=g) / math.sqrt(v * ci)).to(dtype)
    bias = torch.randn(co, generator=g).to(dtype)
    grad = torch.randn(l, co, generator=g).to(dtype)
    fwd_np, bwd_np = sc.neighbor_maps(coords_np, oc_np, tuple(shape), ks, st, pd, dl)
    w5 = weight.double().reshape(co, *ks, ci)
    ref_out = sc.forward(feats.double(), fwd_np, w5, bias.double())
    ref_gi, ref_gw, ref_gb = sc.backward(grad.double(), feats.double(), fwd_np, bwd_np, w5)
    ref_gw = ref_gw.reshape(co, v, ci)

    coords = torch.from_numpy(coords_np).to(dev)
    out_coords = torch.from_numpy(oc_np).to(dev)
    cache = SparseConv3dFunction._compute_neighbor_cache(coords, out_coords, shape, ks, st, pd, dl, True)
    f = feats.to(dev).requires_grad_(True)
    w = weight.to(dev).requires_grad_(True)
    b = bias.to(dev).requires_grad_(True)
    go = grad.to(dev)
    nmap, nmap_bwd = cache["neighbor_map"], cache["neighbor_map_bwd"]

    for tag in ("", "_splitk"):
        _say(f"generic geom={geom} {dtype} non-masked{tag}")
        out = getattr(kernels.triton, "sparse_conv_fwd_implicit_gemm" + tag)(f, w, b, nmap)
        assert tuple(out.shape) == (l, co)
        _close(out, ref_out, dtype, "forward")
        gi, gw, gb = getattr(kernels.triton, "sparse_conv_bwd_implicit_gemm" + tag)(go, f, w, b, nmap, nmap_bwd)
        assert tuple(gi.shape) == (m, ci) and tuple(gw.shape) == (co, v, ci)
        _close(gi, ref_gi, dtype, "dgrad"), _close(gw, ref_gw, dtype, "wgrad"), _close(gb, ref_gb, dtype, "dbias")

        _say(f"generic geom={geom} {dtype} masked{tag}")
        out = getattr(kernels.triton, "sparse_conv_fwd_masked_implicit_gemm" + tag)(
            f, w, b, nmap, cache["sorted_idx"], cache.valid_kernel_callback, cache.valid_kernel_seg_callback)
        _close(out, ref_out, dtype, "forward")
        gi, gw, gb = getattr(kernels.triton, "sparse_conv_bwd_masked_implicit_gemm" + tag)(
            go, f, w, b, nmap, nmap_bwd, cache["valid_signal_i"], cache["valid_signal_o"], cache["valid_signal_seg"],
            cache["sorted_idx_bwd"], cache.valid_kernel_bwd_callback, cache.valid_kernel_bwd_seg_callback)
        _close(gi, ref_gi, dtype, "dgrad"), _close(gw, ref_gw, dtype, "wgrad"), _close(gb, ref_gb, dtype, "dbias")

    # the reference's own way to the input gradient: the forward kernel over the backward map with TRANSPOSE_WEIGHT
    gi = kernels.triton.sparse_conv_fwd_implicit_gemm_splitk(go, w.detach(), None, nmap_bwd, TRANSPOSE_WEIGHT=True)
    _close(gi, ref_gi, dtype, "dgrad through TRANSPOSE_WEIGHT")
    if cache["sorted_idx_bwd"] is not None:
        gi = kernels.triton.sparse_conv_fwd_masked_implicit_gemm_splitk(go, w.detach(), None, nmap_bwd, cache["sorted_idx_bwd"],
                                                                        None, None, TRANSPOSE_WEIGHT=True)
        _close(gi, ref_gi, dtype, "masked dgrad through TRANSPOSE_WEIGHT")


@pytest.mark.gpu
def test_wrong_dtypes_and_shapes_are_refused_before_any_launch(gpu_device):
    """Tables of the wrong element type would be read out of bounds by the kernels: the wrappers refuse them on the host."""
    res, c = 8, 32
    coords = torch.from_numpy(reference_test_shell(res)).to(gpu_device)
    shape = torch.Size([1, c, res, res, res])
    cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
    n = coords.shape[0]
    x = torch.randn(n, c, device=gpu_device).half()
    w = torch.randn(c, 27, c, device=gpu_device).half()
    nmap = cache["neighbor_map"]
    with pytest.raises(AssertionError):     # sorted_idx must be int64
        kernels.triton.sparse_submanifold_conv_fwd_masked_implicit_gemm(x, w, None, nmap, cache["sorted_idx"].int())
    with pytest.raises(AssertionError):     # neighbor must be uint32
        kernels.triton.sparse_submanifold_conv_fwd_implicit_gemm(x, w, None, nmap.view(torch.int32))
    with pytest.raises(AssertionError):     # weight [Co, V, Ci] with the map's V
        kernels.triton.sparse_submanifold_conv_fwd_implicit_gemm(x, w[:, :8].contiguous(), None, nmap)
    with pytest.raises(AssertionError):     # pair lists must be uint32
        kernels.triton.sparse_submanifold_conv_bwd_masked_implicit_gemm(
            x, x.clone().requires_grad_(True), w.requires_grad_(True), None, nmap, cache["sorted_idx"], None, None,
            cache["valid_signal_i"].view(torch.int32), cache["valid_signal_o"], cache["valid_signal_seg"])
    with pytest.raises(ValueError):         # a segment table that names more pairs than the lists hold
        kernels.triton.sparse_submanifold_conv_bwd_masked_implicit_gemm(
            x, x.clone().requires_grad_(True), w.requires_grad_(True), None, nmap.clone(), cache["sorted_idx"], None, None,
            cache["valid_signal_i"][:10].contiguous(), cache["valid_signal_o"][:10].contiguous(), cache["valid_signal_seg"])
    with pytest.raises(AssertionError):
        kernels.cuda.neighbor_map_post_process_for_masked_implicit_gemm_2(cache["gray_code"], cache["sorted_idx"].int(), 64)
    with pytest.raises(AssertionError):
        kernels.cuda.neighbor_map_post_process_for_masked_implicit_gemm_1(nmap.view(torch.int32))
