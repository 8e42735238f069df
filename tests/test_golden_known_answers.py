"""The oracle (CPU) and the HIP path (GPU) against tests/golden/known_answers.json: values that come from neither."""
import json
import os

import numpy as np
import pytest
import torch

from flexgemm_amd.workloads import shell_coords
from oracle import definitions as od
from oracle import neighbor as nb
from oracle import serialize as oz
from oracle import sparse_conv as sc

with open(os.path.join(os.path.dirname(__file__), "golden", "known_answers.json")) as fh:
    KA = json.load(fh)
EMPTY = 0xFFFFFFFF


def test_hash_finalizers():
    for k, want in KA["murmur3_finalizers"]["fmix32"].items():
        assert nb.fmix32(int(k)) == int(want, 16)
    for k, want in KA["murmur3_finalizers"]["fmix64"].items():
        assert nb.fmix64(int(k)) == int(want, 16)


@pytest.mark.parametrize("row", [r for r in KA["benchmark_shells"]["rows"] if r["res"] <= 256], ids=lambda r: f"res{r['res']}")
def test_oracle_counts_of_the_benchmark_shells(row):
    res = row["res"]
    coords = shell_coords(res)
    assert len(coords) == row["voxels"]
    nmap = nb.neighbor_map(coords, (1, 1, res, res, res), (3, 3, 3), (1, 1, 1))
    assert int((nmap != EMPTY).sum()) == row["pairs"]
    assert np.array_equal(nmap[:, 13], np.arange(len(coords), dtype=np.uint32))


def test_curve_codes():
    z = KA["z_order"]
    coords = np.array(z["coords_bxyz"], dtype=np.int32)
    assert oz.encode(coords, z["bit_length"], "z_order").tolist() == z["codes"]
    assert np.array_equal(oz.decode(np.array(z["codes"], dtype=np.int64), z["bit_length"], "z_order"), coords)
    walk = np.array([[0] + p for p in KA["hilbert_first_order"]["walk_xyz"]], dtype=np.int32)
    assert oz.encode(walk, 1, "hilbert").tolist() == list(range(8))
    assert np.array_equal(oz.decode(np.arange(8, dtype=np.int64), 1, "hilbert"), walk)
    # second order: the orientation of the sub-cubes below the first level, worked by hand from Skilling's steps
    second = KA["hilbert_second_order"]
    pts = np.array([[0] + p for p in second["coords_xyz"]], dtype=np.int32)
    assert oz.encode(pts, second["bit_length"], "hilbert").tolist() == second["codes"]
    assert np.array_equal(oz.decode(np.array(second["codes"], dtype=np.int64), second["bit_length"], "hilbert"), pts)


def test_gray_decode_and_output_extent():
    pairs = np.array(KA["gray_decode"]["pairs"], dtype=np.int64)
    assert od.gray_to_binary(pairs[:, 0].astype(np.int32)).tolist() == pairs[:, 1].tolist()
    for n, k, s, p, d, want in KA["output_extent"]["rows"]:
        assert sc.out_dims((1, 1, n, n, n), (k, k, k), (s, s, s), (p, p, p), (d, d, d)) == (want, want, want)


@pytest.mark.gpu
@pytest.mark.parametrize("row", KA["benchmark_shells"]["rows"], ids=lambda r: f"res{r['res']}")
def test_hip_counts_of_the_benchmark_shells(gpu_device, row):
    """Full-size end-to-end check of the table builders: the number of valid (voxel, offset) pairs the HIP neighbor
    cache finds on each benchmark shell, under both ways of finding the neighbors."""
    import flex_gemm
    from flex_gemm.ops.spconv import SubMConv3dFunction
    res = row["res"]
    coords_np = shell_coords(res)
    assert len(coords_np) == row["voxels"]
    coords = torch.from_numpy(coords_np).to(gpu_device)
    print(f"[case] shell counts res={res}", flush=True)
    try:
        for builder in ("hash", "sort"):
            flex_gemm.ops.spconv.set_neighbor_map_builder(builder)
            cache = SubMConv3dFunction._compute_neighbor_cache(coords, torch.Size([1, 8, res, res, res]), (3, 3, 3), (1, 1, 1), True)
            seg = cache.valid_signal_seg.view(torch.int32).cpu().numpy().astype(np.int64) & 0xFFFFFFFF
            assert int(seg[-1]) == row["pairs"], builder
            assert int((cache.neighbor_map.view(torch.int32) != -1).sum()) == row["pairs"], builder
            assert cache.valid_signal_i.shape[0] == row["pairs"] and cache.valid_signal_o.shape[0] == row["pairs"]
    finally:
        flex_gemm.ops.spconv.set_neighbor_map_builder("auto")


@pytest.mark.gpu
def test_hip_curve_codes(gpu_device):
    from flex_gemm import ops
    z = KA["z_order"]
    coords = torch.tensor(z["coords_bxyz"], dtype=torch.int32, device=gpu_device)
    shape = torch.Size([3, 0, 1 << z["bit_length"], 2, 2])
    codes = ops.serialize.encode_seq(coords, shape, mode="z_order")
    assert codes.cpu().tolist() == z["codes"]
    walk = torch.tensor([[0] + p for p in KA["hilbert_first_order"]["walk_xyz"]], dtype=torch.int32, device=gpu_device)
    assert ops.serialize.encode_seq(walk, torch.Size([1, 0, 2, 2, 2]), mode="hilbert").cpu().tolist() == list(range(8))
    second = KA["hilbert_second_order"]
    pts = torch.tensor([[0] + p for p in second["coords_xyz"]], dtype=torch.int32, device=gpu_device)
    assert ops.serialize.encode_seq(pts, torch.Size([1, 0, 4, 4, 4]), mode="hilbert").cpu().tolist() == second["codes"]
