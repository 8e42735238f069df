"""`flex_gemm.kernels.cuda` under the reference's own names (flex_gemm/kernels/cuda/ext.cpp:10-36): the calls the
reference's tests and operators make on its native module give, on the GPU, what the CPU restatements give."""
import sys

import numpy as np
import pytest
import torch

from flex_gemm import kernels
from flexgemm_amd.workloads import reference_test_shell
from oracle import neighbor as nb
from oracle import serialize as ser
from oracle import sparse_conv as sc

REFERENCE_NAMES = [
    "hashmap_insert", "hashmap_lookup", "hashmap_insert_3d", "hashmap_lookup_3d", "hashmap_insert_3d_idx_as_val",
    "z_order_encode", "z_order_decode", "hilbert_encode", "hilbert_decode",
    "hashmap_build_grid_sample_3d_nearest_neighbor_map", "hashmap_build_grid_sample_3d_trilinear_neighbor_map_weight",
    "hashmap_build_submanifold_conv_neighbour_map", "hashmap_build_sparse_conv_out_coords",
    "expand_unique_build_sparse_conv_out_coords", "hashmap_build_sparse_conv_neighbour_map",
    "neighbor_map_post_process_for_masked_implicit_gemm_1_no_bwd", "neighbor_map_post_process_for_masked_implicit_gemm_1",
    "neighbor_map_post_process_for_masked_implicit_gemm_2",
]


def _say(msg):
    print(f"[kernels.cuda] {msg}", file=sys.stderr, flush=True)


def _np(t):
    return t.detach().cpu().numpy()


def _u32(t):
    return _np(t.view(torch.int32)).view(np.uint32)


def test_every_pybind_name_is_there():
    for name in REFERENCE_NAMES:
        assert callable(getattr(kernels.cuda, name)), name


def test_host_tensors_and_grid_sample_are_refused():
    with pytest.raises(NotImplementedError):
        kernels.cuda.z_order_decode(torch.zeros(4, dtype=torch.int32), 4)
    with pytest.raises(NotImplementedError):
        kernels.cuda.hashmap_build_grid_sample_3d_nearest_neighbor_map()
    with pytest.raises(NotImplementedError):
        kernels.cuda.hashmap_build_grid_sample_3d_trilinear_neighbor_map_weight()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype_key", [torch.uint32, torch.uint64])
@pytest.mark.parametrize("dtype_value", [torch.uint32, torch.uint64])
def test_hashmap_round_trip_as_the_reference_runs_it(gpu_device, dtype_key, dtype_value):
    # tests/hashmap.py:13-69: table of 2N slots filled with the key type's maximum, random values in, the same values out
    for res in (1, 2, 4, 16, 64, 128):
        _say(f"hash round trip res={res} key={dtype_key} value={dtype_value}")
        coords = torch.from_numpy(reference_test_shell(res)).to(gpu_device)
        n = coords.shape[0]
        hashmap_keys = torch.full((2 * n,), torch.iinfo(dtype_key).max, dtype=dtype_key, device=gpu_device)
        hashmap_values = torch.empty((2 * n,), dtype=dtype_value, device=gpu_device)
        values = torch.randint(0, torch.iinfo(dtype_value).max // 2, (n,), device=gpu_device).to(dtype_value)
        kernels.cuda.hashmap_insert_3d(hashmap_keys, hashmap_values, coords, values, res, res, res)
        values_ = kernels.cuda.hashmap_lookup_3d(hashmap_keys, hashmap_values, coords, res, res, res)
        assert values_.dtype == dtype_value
        assert torch.equal(values_.view(torch.int64 if dtype_value == torch.uint64 else torch.int32),
                           values.view(torch.int64 if dtype_value == torch.uint64 else torch.int32))

        # pre-serialised keys through the generic pair of calls
        flat = ((coords[:, 0].long() * res + coords[:, 1]) * res + coords[:, 2]) * res + coords[:, 3]
        keys = flat.to(torch.int32).view(torch.uint32) if dtype_key == torch.uint32 else flat.view(torch.uint64)
        hashmap_keys.view(torch.int64 if dtype_key == torch.uint64 else torch.int32).fill_(-1)
        kernels.cuda.hashmap_insert(hashmap_keys, hashmap_values, keys, values)
        again = kernels.cuda.hashmap_lookup(hashmap_keys, hashmap_values, keys)
        assert torch.equal(again.view(torch.int64 if dtype_value == torch.uint64 else torch.int32),
                           values.view(torch.int64 if dtype_value == torch.uint64 else torch.int32))


@pytest.mark.gpu
def test_idx_as_val_then_lookup_gives_row_numbers(gpu_device):
    res = 32
    coords = torch.from_numpy(reference_test_shell(res)).to(gpu_device)
    n = coords.shape[0]
    hashmap_keys = torch.full((2 * n,), torch.iinfo(torch.uint32).max, dtype=torch.uint32, device=gpu_device)
    hashmap_values = torch.empty((2 * n,), dtype=torch.uint32, device=gpu_device)
    kernels.cuda.hashmap_insert_3d_idx_as_val(hashmap_keys, hashmap_values, coords, res, res, res)
    rows = kernels.cuda.hashmap_lookup_3d(hashmap_keys, hashmap_values, coords, res, res, res)
    assert np.array_equal(_u32(rows), np.arange(n, dtype=np.uint32))
    outside = torch.tensor([[0, res, 0, 0], [0, 0, -1, 0]], dtype=torch.int32, device=gpu_device)
    assert (_u32(kernels.cuda.hashmap_lookup_3d(hashmap_keys, hashmap_values, outside, res, res, res)) == 0xFFFFFFFF).all()


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["z_order", "hilbert"])
@pytest.mark.parametrize("bit_length,dtype", [(7, torch.int32), (10, torch.int32), (10, torch.int64), (16, torch.int64)])
def test_curve_codes_by_their_native_names(gpu_device, mode, bit_length, dtype):
    # the call pattern of flex_gemm/ops/serialize.py:35-39, 68-70
    rng = np.random.default_rng(bit_length)
    n = 5000
    coords_np = rng.integers(0, 1 << bit_length, size=(n, 4), dtype=np.int64).astype(np.int32)
    batch_bits = min(2, (32 if dtype == torch.int32 else 64) - 3 * bit_length)
    coords_np[:, 0] = rng.integers(0, 1 << batch_bits, size=n)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    codes = torch.empty((n,), dtype=dtype, device=gpu_device)
    encode = kernels.cuda.z_order_encode if mode == "z_order" else kernels.cuda.hilbert_encode
    decode = kernels.cuda.z_order_decode if mode == "z_order" else kernels.cuda.hilbert_decode
    encode(coords, bit_length, codes)
    want = ser.encode(coords_np, bit_length, mode, np.int32 if dtype == torch.int32 else np.int64)
    assert np.array_equal(_np(codes), want)
    back = decode(codes, bit_length)
    assert back.dtype == torch.int32 and tuple(back.shape) == (n, 4)
    assert np.array_equal(_np(back), coords_np)


@pytest.mark.gpu
def test_submanifold_tables_by_their_native_names(gpu_device):
    # the sequence of flex_gemm/ops/spconv/submanifold_conv3d.py:44-88 on the native module
    res = 48
    coords_np = reference_test_shell(res)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    n = coords.shape[0]
    hashmap_keys = torch.full((2 * n,), torch.iinfo(torch.uint32).max, dtype=torch.uint32, device=gpu_device)
    hashmap_vals = torch.empty((2 * n,), dtype=torch.uint32, device=gpu_device)
    nmap = kernels.cuda.hashmap_build_submanifold_conv_neighbour_map(hashmap_keys, hashmap_vals, coords, res, res, res,
                                                                      3, 3, 3, 1, 1, 1)
    want = nb.neighbor_cache(coords_np, (1, 8, res, res, res), needs_grad=True, blocks=(64,))
    assert nmap.dtype == torch.uint32 and np.array_equal(_u32(nmap), want["neighbor_map"])

    gray, order = kernels.cuda.neighbor_map_post_process_for_masked_implicit_gemm_1_no_bwd(nmap)
    assert np.array_equal(_np(gray), want["gray_code"])
    assert np.array_equal(_np(order), want["sorted_idx"])

    gray2, order2, sig_i, sig_o, seg = kernels.cuda.neighbor_map_post_process_for_masked_implicit_gemm_1(nmap)
    assert torch.equal(gray2, gray) and torch.equal(order2, order)
    assert np.array_equal(_u32(sig_i), want["valid_signal_i"].view(np.uint32))
    assert np.array_equal(_u32(sig_o), want["valid_signal_o"].view(np.uint32))
    assert np.array_equal(_u32(seg), want["valid_signal_seg"].view(np.uint32))

    vk, vk_seg = kernels.cuda.neighbor_map_post_process_for_masked_implicit_gemm_2(gray, order, 64)
    assert np.array_equal(_np(vk), want["valid_kernel_64"])
    assert np.array_equal(_np(vk_seg), want["valid_kernel_seg_64"])


@pytest.mark.gpu
@pytest.mark.parametrize("serialize_mode", [0, 1, 2])
def test_generic_conv_tables_by_their_native_names(gpu_device, serialize_mode):
    # the sequence of flex_gemm/ops/spconv/sparse_conv3d.py:60-94, 119-135 on the native module
    res = 32
    coords_np = reference_test_shell(res)
    coords = torch.from_numpy(coords_np).to(gpu_device)
    geom = (1, res, res, res, 3, 3, 3, 2, 2, 2, 1, 1, 1, 1, 1, 1)
    a = kernels.cuda.hashmap_build_sparse_conv_out_coords(coords, 1.1, serialize_mode, *geom)
    b = kernels.cuda.expand_unique_build_sparse_conv_out_coords(coords, serialize_mode, *geom)
    assert torch.equal(a, b)
    want = sc.output_coords(coords_np, (1, 8, res, res, res), (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1))
    if serialize_mode:
        bit_length = ser.bit_lengths((1, 8, res, res, res))[0]
        want = ser.reorder_coords(want, bit_length, "z_order" if serialize_mode == 1 else "hilbert")
    assert np.array_equal(_np(a), want)

    fwd, bwd = kernels.cuda.hashmap_build_sparse_conv_neighbour_map(coords, a, 2.0, True, *geom)
    want_fwd, want_bwd = sc.neighbor_maps(coords_np, want, (1, 8, res, res, res), (3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1))[:2]
    assert np.array_equal(_u32(fwd), np.asarray(want_fwd).view(np.uint32))
    assert np.array_equal(_u32(bwd), np.asarray(want_bwd).view(np.uint32))
    fwd_only, none = kernels.cuda.hashmap_build_sparse_conv_neighbour_map(coords, a, 2.0, False, *geom)
    assert torch.equal(fwd_only.view(torch.int32), fwd.view(torch.int32)) and none.numel() == 0
