"""GPU parity of the space-filling-curve codes (z-order, Hilbert): bit-exact against the oracle, the reference's own
round-trip sweep (tests/serialize.py:10-66: decode(encode(coords)) == coords for res 1 .. 2048), and the curve orders
of the generic convolution's output coordinates (SerializationMode.Z_ORDER / HILBERT).
"""
import math
import sys

import numpy as np
import pytest
import torch

import flex_gemm
from flex_gemm import ops
from flex_gemm.ops.spconv import SerializationMode, SparseConv3dFunction, sparse_conv3d
from flexgemm_amd.workloads import reference_test_shell
from oracle import serialize as oz
from oracle import sparse_conv as sc

pytestmark = pytest.mark.gpu
MODES = ["z_order", "hilbert"]


def _say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def _random_coords(n, batch, res, seed):
    rng = np.random.default_rng(seed)
    return np.concatenate([rng.integers(0, batch, (n, 1)), rng.integers(0, res, (n, 3))], axis=1).astype(np.int32)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("res", [1, 2, 4, 8, 16, 32, 64, 128])
def test_codes_match_oracle_on_the_reference_shell(gpu_device, mode, res):
    coords_np = np.ascontiguousarray(reference_test_shell(res))
    shape = torch.Size([1, 0, res, res, res])
    _say(f"serialize shell res={res} mode={mode} n={len(coords_np)}")
    coords = torch.from_numpy(coords_np).to(gpu_device)
    codes = ops.serialize.encode_seq(coords, shape, mode=mode)
    want = oz.encode_seq(coords_np, shape, mode)
    assert codes.dtype == torch.int32 and codes.shape == (len(coords_np),)
    assert np.array_equal(codes.cpu().numpy(), want)
    back = ops.serialize.decode_seq(codes, shape, mode=mode)
    assert back.dtype == torch.int32 and torch.equal(back, coords)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("batch,res", [(1, 1024), (4, 1024), (5, 1024), (1, 2048), (3, 1 << 16), (2, 1 << 21), (1, 1 << 21)])
def test_random_coords_all_widths(gpu_device, mode, batch, res):
    """32-bit codes up to 32 bits in total (batch 4 at res 1024), 64-bit codes beyond, up to 21 bits per axis."""
    n = 200_000
    coords_np = _random_coords(n, batch, res, seed=batch + res % 1000)
    coords_np[0] = (batch - 1, res - 1, res - 1, res - 1)
    coords_np[1] = (0, 0, 0, 0)
    shape = torch.Size([batch, 0, res, 7, res // 2 or 1])
    _say(f"serialize random batch={batch} res={res} mode={mode}")
    coords = torch.from_numpy(coords_np).to(gpu_device)
    codes = ops.serialize.encode_seq(coords, shape, mode=mode)
    want = oz.encode_seq(coords_np, shape, mode)
    assert codes.cpu().numpy().dtype == want.dtype
    assert np.array_equal(codes.cpu().numpy(), want)
    assert torch.equal(ops.serialize.decode_seq(codes, shape, mode=mode), coords)
    # decoding is also right for codes the oracle made
    assert torch.equal(ops.serialize.decode_seq(torch.from_numpy(want).to(gpu_device), shape, mode=mode), coords)


@pytest.mark.parametrize("mode", MODES)
def test_round_trip_at_full_size(gpu_device, mode):
    """The reference's largest case is the res-2048 shell (about 10.7 M voxels); the same count of random voxels of that
    grid goes through here, checked by the round trip and by the codes being distinct for distinct voxels."""
    res, n = 2048, 10_700_000
    shape = torch.Size([1, 0, res, res, res])
    g = torch.Generator(device="cpu").manual_seed(7)
    flat = torch.randint(0, res ** 3, (n,), generator=g, dtype=torch.int64).unique()
    coords = torch.stack([torch.zeros_like(flat), flat // (res * res), flat // res % res, flat % res], dim=1).int().to(gpu_device)
    _say(f"serialize full size mode={mode} n={coords.shape[0]}")
    codes = ops.serialize.encode_seq(coords, shape, mode=mode)
    assert codes.dtype == torch.int64
    assert torch.equal(ops.serialize.decode_seq(codes, shape, mode=mode), coords)
    assert torch.unique(codes).numel() == coords.shape[0]
    assert int(codes.min()) >= 0 and int(codes.max()) < 8 ** 11


def test_hilbert_walk_on_device(gpu_device):
    """Decoding 0 .. 8^k - 1 on the device walks the cube one face-adjacent step at a time."""
    k = 5
    shape = torch.Size([1, 0, 1 << k, 1 << k, 1 << k])
    codes = torch.arange(8 ** k, dtype=torch.int32, device=gpu_device)
    walk = ops.serialize.decode_seq(codes, shape, mode="hilbert").cpu().numpy().astype(np.int64)
    assert np.all(walk[:, 0] == 0)
    assert np.all(np.abs(np.diff(walk[:, 1:], axis=0)).sum(axis=1) == 1)
    assert walk[0].tolist() == [0, 0, 0, 0] and walk[-1].tolist() == [0, (1 << k) - 1, 0, 0]


def test_errors_and_empty(gpu_device):
    shape = torch.Size([1, 0, 64, 64, 64])
    coords = torch.zeros((3, 4), dtype=torch.int32, device=gpu_device)
    with pytest.raises(ValueError, match="Unknown encoding mode"):
        ops.serialize.encode_seq(coords, shape, mode="peano")
    with pytest.raises(ValueError, match="Unknown decoding mode"):
        ops.serialize.decode_seq(torch.zeros(3, dtype=torch.int32, device=gpu_device), shape, mode="peano")
    with pytest.raises(ValueError, match="too large"):
        ops.serialize.encode_seq(coords, torch.Size([2, 0, 1 << 22, 4, 4]))
    with pytest.raises(AssertionError):
        ops.serialize.encode_seq(coords[:, :3], shape)
    with pytest.raises(NotImplementedError):
        ops.serialize.encode_seq(coords.cpu(), shape)
    empty = torch.zeros((0, 4), dtype=torch.int32, device=gpu_device)
    for mode in MODES:
        codes = ops.serialize.encode_seq(empty, shape, mode=mode)
        assert codes.shape == (0,) and codes.dtype == torch.int32
        assert ops.serialize.decode_seq(codes, shape, mode=mode).shape == (0, 4)


@pytest.fixture
def serialization_mode():
    def set_mode(mode):
        flex_gemm.ops.spconv.SERIALIZATION_MODE = mode
    yield set_mode
    flex_gemm.ops.spconv.SERIALIZATION_MODE = SerializationMode.BXYZ


GEOMS = [
    ((3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),
    ((2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1)),
    ((3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1)),
]


@pytest.mark.parametrize("mode", [SerializationMode.Z_ORDER, SerializationMode.HILBERT])
@pytest.mark.parametrize("res", [2, 8, 32, 64])
def test_output_coords_follow_the_curve(gpu_device, serialization_mode, mode, res):
    """Same set of output coordinates as under BXYZ, in ascending code order with bits per axis taken from the input
    grid (the rule of the reference's builder, sparse_neighbor_map.cu:157-160)."""
    name = "z_order" if mode == SerializationMode.Z_ORDER else "hilbert"
    for batch in (1, 3):
        coords_np = np.ascontiguousarray(reference_test_shell(res, batch=batch) if batch > 1 else reference_test_shell(res))
        coords_np = coords_np[np.random.default_rng(res).permutation(len(coords_np))]
        shape = torch.Size([batch, 0, res, res, res])
        coords = torch.from_numpy(coords_np).to(gpu_device)
        for ks, st, pd, dl in GEOMS:
            _say(f"curve out coords mode={name} res={res} batch={batch} K={ks} S={st}")
            serialization_mode(mode)
            got = SparseConv3dFunction._get_output_coords(coords, shape, ks, st, pd, dl).cpu().numpy()
            base = sc.output_coords(coords_np, tuple(shape), ks, st, pd, dl)
            want = oz.reorder_coords(base, (res - 1).bit_length(), name)
            assert got.shape == want.shape and np.array_equal(got, want)


@pytest.mark.parametrize("mode", [SerializationMode.Z_ORDER, SerializationMode.HILBERT])
def test_conv_with_curve_ordered_outputs(gpu_device, serialization_mode, mode):
    """The whole operator under a curve mode: rows of the result follow the curve-ordered output coordinates."""
    from oracle import explicit_gemm as eg
    res, ci, co = 24, 32, 48
    name = "z_order" if mode == SerializationMode.Z_ORDER else "hilbert"
    coords_np = np.ascontiguousarray(reference_test_shell(res))
    shape = torch.Size([1, 0, res, res, res])
    ks, st, pd, dl = GEOMS[2]
    g = torch.Generator().manual_seed(11)
    feats = torch.randn(len(coords_np), ci, generator=g).half()
    weight = (torch.randn(co, *ks, ci, generator=g) / math.sqrt(27 * ci)).half()
    bias = torch.randn(co, generator=g).half()
    oc_np = oz.reorder_coords(sc.output_coords(coords_np, tuple(shape), ks, st, pd, dl), (res - 1).bit_length(), name)
    fwd, _ = sc.neighbor_maps(coords_np, oc_np, tuple(shape), ks, st, pd, dl)
    ref = sc.forward(feats.double(), fwd, weight.double(), bias.double())
    serialization_mode(mode)
    _say(f"sparse conv under serialization mode {name}")
    out, oc, _ = sparse_conv3d(feats.to(gpu_device), torch.from_numpy(coords_np).to(gpu_device), shape, weight.to(gpu_device),
                               bias.to(gpu_device), stride=st, padding=pd, dilation=dl)
    assert np.array_equal(oc.cpu().numpy(), oc_np)
    assert eg.max_rel_err(out.cpu(), ref) <= 1e-2          # fp16 tolerance of the operator


def test_curve_mode_rejects_an_output_grid_wider_than_the_input_bits(gpu_device, serialization_mode):
    res = 8
    coords = torch.from_numpy(np.ascontiguousarray(reference_test_shell(res))).to(gpu_device)
    serialization_mode(SerializationMode.HILBERT)
    with pytest.raises(ValueError, match="bits per axis"):
        SparseConv3dFunction._get_output_coords(coords, torch.Size([1, 0, res, res, res]), (3, 3, 3), (1, 1, 1), (2, 2, 2), (1, 1, 1))
