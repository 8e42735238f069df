"""Host-side (CPU) checks of the generic sparse convolution operator: the torch builders and the explicit-GEMM path
against the oracle, and the error behaviour without a GPU.  No device code runs here."""
import math

import numpy as np
import pytest
import torch

import flex_gemm
from flex_gemm.ops.spconv import Algorithm, SparseConv3dFunction, SparseConv3dNeighborCache, sparse_conv3d
from oracle import sparse_conv as sc

GEOMS = [
    ((3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    ((3, 3, 3), (1, 1, 1), (2, 2, 2), (2, 2, 2)),
    ((2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1)),
    ((3, 2, 1), (2, 1, 3), (1, 0, 2), (1, 2, 1)),
]


def _coords(dims, batch, seed):
    g = torch.Generator().manual_seed(seed)
    c = torch.nonzero(torch.rand(batch, *dims, generator=g) < 0.3).int()
    return c[torch.randperm(len(c), generator=g)].contiguous()


def _u32(t):
    return t.view(torch.int32).numpy().view(np.uint32)


@pytest.mark.parametrize("ks,st,pd,dl", GEOMS)
def test_torch_builders_and_explicit_path(ks, st, pd, dl):
    dims = (9, 7, 8)
    shape = torch.Size([2, 0, *dims])
    coords = _coords(dims, 2, 0)
    oc = SparseConv3dFunction._get_output_coords_torch(coords, shape, ks, st, pd, dl)
    oc_np = sc.output_coords(coords.numpy(), tuple(shape), ks, st, pd, dl)
    assert oc.dtype == torch.int32 and np.array_equal(oc.numpy(), oc_np)
    flex_gemm.ops.spconv.set_algorithm(Algorithm.EXPLICIT_GEMM)
    try:
        cache = SparseConv3dFunction._compute_neighbor_cache_torch(coords, oc, shape, ks, st, pd, dl, True)
        fwd, bwd = sc.neighbor_maps(coords.numpy(), oc_np, tuple(shape), ks, st, pd, dl)
        assert np.array_equal(_u32(cache.neighbor_map), fwd) and np.array_equal(_u32(cache.neighbor_map_bwd), bwd)
        assert cache["no_such_field"] is None                       # a missing field reads as None (reference :14-15)
        g = torch.Generator().manual_seed(1)
        ci, co, v = 5, 6, ks[0] * ks[1] * ks[2]
        feats = torch.randn(len(coords), ci, generator=g, dtype=torch.float64).requires_grad_(True)
        weight = (torch.randn(co, *ks, ci, generator=g, dtype=torch.float64) / math.sqrt(v * ci)).requires_grad_(True)
        bias = torch.randn(co, generator=g, dtype=torch.float64).requires_grad_(True)
        grad = torch.randn(len(oc), co, generator=g, dtype=torch.float64)
        out = SparseConv3dFunction._sparse_conv_forward(feats.detach(), cache, weight.detach(), bias.detach())
        assert torch.allclose(out, sc.forward(feats.detach(), fwd, weight.detach(), bias.detach()), rtol=1e-12, atol=1e-12)
        gi, gw, gb = SparseConv3dFunction._sparse_conv_backward(grad, feats, cache, weight, bias)
        ri, rw, rb = sc.backward(grad, feats.detach(), fwd, bwd, weight.detach())
        assert torch.allclose(gi, ri, rtol=1e-12, atol=1e-12) and torch.allclose(gw, rw, rtol=1e-12, atol=1e-12)
        assert torch.allclose(gb, rb, rtol=1e-12, atol=1e-12)
    finally:
        flex_gemm.ops.spconv.set_algorithm(Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)


def test_cpu_tensors_are_refused_where_the_reference_refuses_them():
    coords = _coords((4, 4, 4), 1, 2)
    shape = torch.Size([1, 0, 4, 4, 4])
    with pytest.raises(NotImplementedError):
        SparseConv3dFunction._get_output_coords(coords, shape, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1))
    with pytest.raises(NotImplementedError):
        SparseConv3dFunction._compute_neighbor_cache(coords, coords, shape, (3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1), False)
    with pytest.raises(NotImplementedError):
        sparse_conv3d(torch.zeros(len(coords), 4), coords, shape, torch.zeros(4, 3, 3, 3, 4))
    with pytest.raises(RuntimeError):      # a cache without gradients has no backward map to walk
        SparseConv3dNeighborCache(neighbor_map=torch.zeros((1, 27), dtype=torch.int32), neighbor_map_bwd=None)._bwd_view()
    assert flex_gemm.ops.spconv.SERIALIZATION_MODE == flex_gemm.ops.spconv.SerializationMode.BXYZ
    assert flex_gemm.ops.spconv.OUT_COORD_ALGO == flex_gemm.ops.spconv.SparseConv3dOutCoordAlgorithm.HASHMAP
