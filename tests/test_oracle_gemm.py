"""Pins the explicit gather-GEMM restatement (oracle/explicit_gemm.py) against a library routine
(dense conv3d + autograd), closed forms and invariants.  CPU only."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from flexgemm_amd.workloads import make_workload, reference_test_shell
from oracle import definitions as df
from oracle import explicit_gemm as eg
from oracle import neighbor as nb


def _random_case(res, ci, co, seed, density=0.35, dilation=(1, 1, 1)):
    g = torch.Generator().manual_seed(seed)
    occ = torch.rand(res, res, res, generator=g) < density
    coords = torch.nonzero(occ).int()
    coords = torch.cat([torch.zeros(len(coords), 1, dtype=torch.int32), coords], 1)
    coords = coords[torch.randperm(len(coords), generator=g)].contiguous()
    n = len(coords)
    feats = torch.randn(n, ci, generator=g, dtype=torch.float64)
    weight = torch.randn(co, 3, 3, 3, ci, generator=g, dtype=torch.float64) / math.sqrt(27 * ci)
    bias = torch.randn(co, generator=g, dtype=torch.float64)
    grad = torch.randn(n, co, generator=g, dtype=torch.float64)
    nmap = torch.from_numpy(nb.neighbor_map(coords.numpy(), (1, ci, res, res, res), (3, 3, 3), dilation).view(np.int32))
    return coords, feats, weight, bias, grad, nmap


def _scatter_dense(dense, x, y, z, f):
    """dense[:, x_n, y_n, z_n] = f[n, :] (differentiable)."""
    res = dense.shape[1]
    flat = (x * res + y) * res + z
    return dense.reshape(dense.shape[0], -1).index_copy(1, flat, f.t()).reshape(dense.shape)


@pytest.mark.parametrize("dilation", [(1, 1, 1), (2, 1, 2)])
def test_against_dense_conv3d(dilation):
    res, ci, co = 9, 5, 7
    coords, feats, weight, bias, grad, nmap = _random_case(res, ci, co, 0, dilation=dilation)
    x, y, z = coords[:, 1].long(), coords[:, 2].long(), coords[:, 3].long()
    f = feats.clone().requires_grad_(True)
    w = weight.clone().requires_grad_(True)
    b = bias.clone().requires_grad_(True)
    dense_in = torch.zeros(ci, res, res, res, dtype=torch.float64)
    dense_in = _scatter_dense(dense_in, x, y, z, f)
    # weight [Co, Kw, Kh, Kd, Ci] -> conv3d's [Co, Ci, Kw, Kh, Kd]; cross-correlation, zero padding
    out_dense = F.conv3d(dense_in[None], w.permute(0, 4, 1, 2, 3), b, padding=dilation, dilation=dilation)[0]
    out_ref = out_dense[:, x, y, z].t()
    out_ref.backward(grad)
    out = eg.forward(feats, nmap, weight, bias, chunk_rows=37)
    assert torch.allclose(out, out_ref.detach(), rtol=1e-12, atol=1e-12)
    gi, gw, gb = eg.backward(grad, feats, nmap, weight, chunk_rows=41)
    assert torch.allclose(gi, f.grad, rtol=1e-12, atol=1e-12)
    assert torch.allclose(gw, w.grad, rtol=1e-12, atol=1e-12)
    assert torch.allclose(gb, b.grad, rtol=1e-12, atol=1e-12)


def test_closed_forms_and_invariants():
    res, ci, co = 8, 4, 6
    coords, feats, weight, bias, grad, nmap = _random_case(res, ci, co, 3)
    # single voxel: out = feats @ W[:, centre, :].T + bias
    one = torch.full((1, 27), -1, dtype=torch.int32)
    one[0, 13] = 0
    o = eg.forward(feats[:1], one, weight, bias)
    assert torch.allclose(o, feats[:1] @ weight.reshape(co, 27, ci)[:, 13].t() + bias)
    # all-ones weight, no bias: out[n, :] = sum over present neighbors of sum_ci feats
    ones = torch.ones(co, 3, 3, 3, ci, dtype=torch.float64)
    o = eg.forward(feats, nmap, ones, None)
    idx = nmap.long()
    expect = torch.stack([feats[idx[n][idx[n] >= 0]].sum() for n in range(len(idx))])
    assert torch.allclose(o, expect[:, None].expand(-1, co))
    # linearity in feats and in weight
    f2 = torch.randn_like(feats)
    a = eg.forward(feats + 2 * f2, nmap, weight, None)
    assert torch.allclose(a, eg.forward(feats, nmap, weight, None) + 2 * eg.forward(f2, nmap, weight, None))
    # chunk-size invariance (forward bitwise per row; wgrad up to summation order)
    assert torch.equal(eg.forward(feats, nmap, weight, bias, chunk_rows=7), eg.forward(feats, nmap, weight, bias, chunk_rows=10 ** 6))
    g1 = eg.backward(grad, feats, nmap, weight, chunk_rows=7)
    g2 = eg.backward(grad, feats, nmap, weight, chunk_rows=10 ** 6)
    for x, y in zip(g1, g2):
        assert torch.allclose(x, y, rtol=1e-12, atol=1e-12)
    # adjointness: <conv(f), g> == <f, dgrad(g)> == <W, wgrad(f, g)> (bias-free)
    lhs = (eg.forward(feats, nmap, weight, None) * grad).sum()
    assert torch.allclose(lhs, (feats * g1[0]).sum())
    assert torch.allclose(lhs, (weight * g1[1]).sum())


def test_single_offset_weight_gradient_is_a_slice_of_backward():
    res, ci, co = 9, 5, 7
    coords, feats, weight, bias, grad, nmap = _random_case(res, ci, co, 5)
    gw = eg.backward(grad, feats, nmap, weight, need_input=False, need_bias=False)[1].reshape(co, 27, ci)
    for v in range(27):
        for chunk in (3, 10 ** 6):
            assert torch.allclose(eg.weight_grad_offset(grad, feats, nmap, v, chunk_rows=chunk), gw[:, v], rtol=1e-12, atol=1e-12)
    # the centre offset pairs every row with itself
    assert torch.allclose(eg.weight_grad_offset(grad, feats, nmap, 13), grad.t() @ feats, rtol=1e-12, atol=1e-12)


def test_map_forms_accepted():
    res, ci, co = 6, 3, 3
    coords, feats, weight, bias, grad, nmap = _random_case(res, ci, co, 9)
    a = eg.forward(feats, nmap, weight, bias)
    b = eg.forward(feats, nmap.view(torch.uint32), weight, bias)
    c = eg.forward(feats, torch.where(nmap < 0, torch.tensor(0xFFFFFFFF), nmap.long()), weight, bias)
    assert torch.equal(a, b) and torch.equal(a, c)


def test_cpu_plumbing_config1():
    """Configuration 1: res 64 shell, Ci = Co = 64, fp32, forward through the explicit path on the CPU."""
    wl = make_workload("cfg1")
    assert wl.n == 10208
    nmap = torch.from_numpy(nb.neighbor_map(wl.coords.numpy(), tuple(wl.shape)).view(np.int32))
    assert int((nmap != -1).sum()) == 105488
    out32 = eg.forward(wl.feats, nmap, wl.weight, wl.bias)
    out64 = eg.forward(wl.feats.double(), nmap, wl.weight.double(), wl.bias.double())
    assert out32.dtype == torch.float32 and out32.shape == (10208, 64)
    assert eg.max_rel_err(out32, out64) <= 1e-5
    assert eg.calc_err(out32, out64)[0] <= 1e-4
