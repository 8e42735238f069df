"""Pins the generic sparse-convolution restatement (oracle/sparse_conv.py) against brute force written from the
definition, dense conv3d + autograd with the same stride / padding / dilation, and the submanifold special case.
CPU only."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import neighbor as nb
from oracle import sparse_conv as sc

# (kernel, stride, padding, dilation): the reference's own sweep (tests/spconv/neighbor_cache.py:80-86,
# tests/spconv/out_coords.py:39-42) plus anisotropic and "gappy" settings
CASES = [
    ((3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    ((3, 3, 3), (1, 1, 1), (2, 2, 2), (2, 2, 2)),
    ((2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1)),
    ((3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1)),
    ((3, 2, 1), (2, 1, 3), (1, 0, 2), (1, 2, 1)),
    ((2, 2, 2), (3, 3, 3), (0, 0, 0), (1, 1, 1)),     # stride > kernel: some inputs reach no output
]


def _random_coords(dims, batch, density, seed):
    g = torch.Generator().manual_seed(seed)
    occ = torch.rand(batch, *dims, generator=g) < density
    coords = torch.nonzero(occ).int()
    return coords[torch.randperm(len(coords), generator=g)].contiguous().numpy()


@pytest.mark.parametrize("ks,stride,pad,dil", CASES)
def test_tables_against_bruteforce(ks, stride, pad, dil):
    dims = (7, 6, 9)
    shape = (2, 4, *dims)
    coords = _random_coords(dims, 2, 0.3, 1)
    oc = sc.output_coords(coords, shape, ks, stride, pad, dil)
    assert oc.dtype == np.int32
    assert np.array_equal(oc, sc.output_coords_bruteforce(coords, shape, ks, stride, pad, dil))
    fwd, bwd = sc.neighbor_maps(coords, oc, shape, ks, stride, pad, dil)
    fwd_b, bwd_b = sc.neighbor_maps_bruteforce(coords, oc, shape, ks, stride, pad, dil)
    assert np.array_equal(fwd, fwd_b) and np.array_equal(bwd, bwd_b)
    # every output row found at least one input (that is what put it on the list), and the two maps are transposes
    assert (fwd != sc.EMPTY).any(axis=1).all()
    o, v = np.nonzero(fwd != sc.EMPTY)
    assert np.array_equal(bwd[fwd[o, v], v], o.astype(np.uint32))
    assert (bwd != sc.EMPTY).sum() == len(o)
    # user-given output coordinates: a shuffled subset plus cells nobody reaches
    wo, ho, do = sc.out_dims(shape, ks, stride, pad, dil)
    rng = np.random.default_rng(0)
    extra = np.stack([rng.integers(0, 2, 5), rng.integers(0, wo, 5), rng.integers(0, ho, 5), rng.integers(0, do, 5)], 1).astype(np.int32)
    given = np.unique(np.concatenate([oc[rng.permutation(len(oc))[: max(1, len(oc) // 2)]], extra]), axis=0)
    given = given[rng.permutation(len(given))]
    fwd, bwd = sc.neighbor_maps(coords, given, shape, ks, stride, pad, dil)
    fwd_b, bwd_b = sc.neighbor_maps_bruteforce(coords, given, shape, ks, stride, pad, dil)
    assert np.array_equal(fwd, fwd_b) and np.array_equal(bwd, bwd_b)


def test_empty_inputs():
    shape = (1, 4, 5, 5, 5)
    none = np.empty((0, 4), dtype=np.int32)
    assert sc.output_coords(none, shape, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)).shape == (0, 4)
    fwd, bwd = sc.neighbor_maps(none, none, shape, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1))
    assert fwd.shape == (0, 27) and bwd.shape == (0, 27)


def test_reduces_to_submanifold_map():
    dims = (8, 8, 8)
    shape = (1, 4, *dims)
    coords = _random_coords(dims, 1, 0.4, 2)
    fwd, bwd = sc.neighbor_maps(coords, coords, shape, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1))
    subm = nb.neighbor_map(coords, shape, (3, 3, 3), (1, 1, 1))
    assert np.array_equal(fwd, subm)
    assert np.array_equal(bwd, subm[:, ::-1])       # the reference's submanifold backward flips the map instead


@pytest.mark.parametrize("ks,stride,pad,dil", CASES)
def test_against_dense_conv3d(ks, stride, pad, dil):
    dims = (7, 6, 9)
    ci, co, batch = 3, 5, 2
    shape = (batch, ci, *dims)
    coords = _random_coords(dims, batch, 0.3, 4)
    g = torch.Generator().manual_seed(9)
    m = len(coords)
    v = ks[0] * ks[1] * ks[2]
    feats = torch.randn(m, ci, generator=g, dtype=torch.float64)
    weight = torch.randn(co, *ks, ci, generator=g, dtype=torch.float64) / math.sqrt(v * ci)
    bias = torch.randn(co, generator=g, dtype=torch.float64)
    oc = sc.output_coords(coords, shape, ks, stride, pad, dil)
    fwd, bwd = sc.neighbor_maps(coords, oc, shape, ks, stride, pad, dil)
    grad = torch.randn(len(oc), co, generator=g, dtype=torch.float64)

    f = feats.clone().requires_grad_(True)
    w = weight.clone().requires_grad_(True)
    b = bias.clone().requires_grad_(True)
    c = torch.from_numpy(coords).long()
    # channels-last dense grid, filled differentiably, then moved to conv3d's [B, Ci, W, H, D]
    dense = torch.zeros(batch, *dims, ci, dtype=torch.float64).index_put((c[:, 0], c[:, 1], c[:, 2], c[:, 3]), f)
    dense = dense.permute(0, 4, 1, 2, 3)
    out_dense = F.conv3d(dense, w.permute(0, 4, 1, 2, 3), b, stride=stride, padding=pad, dilation=dil)
    assert tuple(out_dense.shape[2:]) == sc.out_dims(shape, ks, stride, pad, dil)
    o = torch.from_numpy(oc).long()
    out_ref = out_dense[o[:, 0], :, o[:, 1], o[:, 2], o[:, 3]]
    # cells off the list see no input: the dense result there is the bias alone
    off = torch.ones(out_dense.shape[0], *out_dense.shape[2:], dtype=torch.bool)
    off[o[:, 0], o[:, 1], o[:, 2], o[:, 3]] = False
    assert torch.allclose(out_dense.detach().permute(0, 2, 3, 4, 1)[off], bias.expand(int(off.sum()), co), rtol=0, atol=1e-13)
    out_ref.backward(grad)

    out = sc.forward(feats, fwd, weight, bias)
    assert torch.allclose(out, out_ref.detach(), rtol=1e-12, atol=1e-12)
    gi, gw, gb = sc.backward(grad, feats, fwd, bwd, weight)
    assert torch.allclose(gi, f.grad, rtol=1e-12, atol=1e-12)
    assert torch.allclose(gw, w.grad, rtol=1e-12, atol=1e-12)
    assert torch.allclose(gb, b.grad, rtol=1e-12, atol=1e-12)
