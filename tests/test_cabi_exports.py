"""The C-ABI library builds, loads and exports every symbol include/flexgemm_hip.h declares (CPU only:
no compute call is made)."""
import ctypes
import os
import re

import pytest

from flexgemm_amd import _native as nat

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "flexgemm_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fgx_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def library():
    if not os.path.exists(nat.lib_path()):
        from flexgemm_amd import build
        build.build(verbose=False)
    return ctypes.CDLL(nat.lib_path())


@pytest.mark.parametrize("compiler,flags", [("gcc", ["-std=c99", "-x", "c"]), ("g++", ["-std=c++17", "-x", "c++"])])
def test_header_is_plain_c_and_cxx(compiler, flags):
    """The boundary is a C ABI: the header must compile on its own as pedantic C99 (what cgo / ctypes-style bindings see)
    and as C++, without HIP or torch headers on the include path."""
    import shutil
    import subprocess
    if shutil.which(compiler) is None:
        pytest.skip(f"{compiler} is not installed")
    header = os.path.join(ROOT, "include", "flexgemm_hip.h")
    done = subprocess.run([compiler, *flags, "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", header],
                          capture_output=True, text=True)
    assert done.returncode == 0, done.stderr


def test_host_program_is_built_beside_the_library(library):
    """The torch-free caller of the C ABI that the GPU tests run links against the in-tree library and nothing of Python."""
    import subprocess
    from flexgemm_amd import build
    if not os.path.exists(build.HOST_CHECK):
        build.build(verbose=False)
    needed = subprocess.run(["ldd", build.HOST_CHECK], capture_output=True, text=True).stdout
    assert "libflexgemm_hip.so" in needed and "torch" not in needed and "python" not in needed.lower()


def test_header_and_binding_agree():
    assert _declared_symbols() == sorted(nat.EXPORTS)


def test_every_declared_symbol_is_exported(library):
    for name in _declared_symbols():
        assert hasattr(library, name), name


def test_host_only_entry_points(library):
    # these touch no device: identity, sizing and the schedule table
    assert library.fgx_abi_version() == 2
    L = nat.lib()
    import torch
    s = nat.table_lookup(nat.PASS_FWD, torch.float16, 669288, 128, 128, 27)
    assert s.tile_rows in (128, 256) and s.tile_cols == 128 and s.splitk == 1 and s.slab_bytes in (64, 128)
    # the persistent streaming kernel walks 256-row tiles; rows of 128 bytes or more use 128-byte K-slabs
    assert (s.stream, s.tile_rows, s.slab_bytes) in ((1, 256, 128), (0, s.tile_rows, s.slab_bytes))
    # a weight of one 128 x 128 tile: the sweep (stream 2, block_rows = its sub-block size)
    s = nat.table_lookup(nat.PASS_WGRAD, torch.float16, 669288, 128, 128, 27)
    assert s.block_rows >= 1024 and s.stream == 2 and (s.tile_rows, s.tile_cols) == (128, 128)
    s = nat.table_lookup(nat.PASS_WGRAD, torch.bfloat16, 40000, 48, 64, 27)
    assert s.stream == 2 and (s.tile_rows, s.tile_cols) == (64, 64)
    # ... not for several tiles, 32 x 32 tiles, few voxels, more than 2^24 of them, or fp32
    s = nat.table_lookup(nat.PASS_WGRAD, torch.float16, 669288, 256, 128, 27)
    assert s.stream == 1 and (s.tile_rows, s.tile_cols) == (128, 256)          # wide on the input side only
    s = nat.table_lookup(nat.PASS_WGRAD, torch.float16, 669288, 128, 384, 27)
    assert s.stream == 1 and (s.tile_rows, s.tile_cols) == (128, 128)          # 384 rows: 256-row tiles would pad more
    assert nat.table_lookup(nat.PASS_WGRAD, torch.float16, 669288, 32, 32, 27).stream == 1
    assert nat.table_lookup(nat.PASS_WGRAD, torch.float16, 4000, 128, 128, 27).stream == 1
    assert nat.table_lookup(nat.PASS_WGRAD, torch.float16, (1 << 24) + 1, 128, 128, 27).stream == 1
    # the table answers stream = 2 up to 2^24 rows; the host falls back to the block-major kernel where the sweep's own
    # limits (operands and pair lists below 0xFF000000 bytes) are tighter than that
    from flexgemm_amd.ops.spconv.submanifold_conv3d import _sweep_fits
    n_big = 16_711_681                                     # x 128 channels x 2 bytes: just past 0xFF000000
    assert nat.table_lookup(nat.PASS_WGRAD, torch.float16, n_big, 128, 128, 27).stream == 2
    assert not _sweep_fits(n_big, n_big, 128, 128, 2, 27 * 1000)
    assert _sweep_fits(n_big - 1, n_big - 1, 128, 128, 2, 27 * 1000)
    assert _sweep_fits(669288, 669288, 128, 128, 2, 7082928)
    assert not _sweep_fits(669288, 669288, 128, 128, 2, 0)                    # no pairs: nothing to sweep
    assert not _sweep_fits((1 << 24) + 1, 100, 64, 64, 2, 1000)                # 24-bit row numbers
    assert not _sweep_fits(1 << 24, 1 << 24, 64, 64, 2, (0xFF000000 - 256) // 4 + 1)   # pair lists past the offset range
    assert nat.table_lookup(nat.PASS_WGRAD, torch.float32, 669288, 128, 128, 27).stream == 0
    s = nat.table_lookup(nat.PASS_FWD, torch.float32, 100, 16, 16, 27)
    assert s.tile_rows in (32, 64, 128) and s.tile_cols == 32 and s.splitk >= 1 and s.stream == 0
    # rule (no table entry): big problems stream, small ones and rows below 64 bytes do not
    s = nat.table_lookup(nat.PASS_DGRAD, torch.bfloat16, 300000, 192, 160, 27)      # 192 input-gradient columns: one wide tile
    assert (s.stream, s.tile_rows, s.tile_cols, s.slab_bytes, s.splitk) == (1, 128, 256, 128, 1)
    s = nat.table_lookup(nat.PASS_FWD, torch.bfloat16, 300000, 192, 320, 27)        # beyond 256 columns: 256-row tiles
    assert (s.stream, s.tile_rows, s.tile_cols, s.slab_bytes, s.splitk) == (1, 256, 128, 128, 1)
    s = nat.table_lookup(nat.PASS_FWD, torch.float16, 166232, 256, 256, 27)         # (a table entry)
    assert (s.stream, s.tile_rows, s.tile_cols, s.slab_bytes, s.splitk) == (1, 128, 256, 128, 1)
    s = nat.table_lookup(nat.PASS_FWD, torch.bfloat16, 300000, 32, 32, 27)      # 64-byte rows: 64-byte slabs, 32-column tiles
    assert (s.stream, s.tile_rows, s.tile_cols, s.slab_bytes, s.splitk) == (1, 256, 32, 64, 1)
    s = nat.table_lookup(nat.PASS_DGRAD, torch.bfloat16, 300000, 96, 32, 27)    # K = Co = 32, 96 input-gradient columns
    assert (s.stream, s.tile_rows, s.tile_cols, s.slab_bytes) == (1, 256, 128, 64)
    assert nat.table_lookup(nat.PASS_FWD, torch.float16, 300000, 16, 64, 27).stream == 0
    assert nat.table_lookup(nat.PASS_FWD, torch.float16, 300000, 128, 32, 27).stream == 0   # no 32-column tile for long rows
    s = nat.table_lookup(nat.PASS_FWD, torch.float16, 300000, 64, 64, 27)       # 128-byte rows of a 16-bit type: 64-byte slabs
    assert (s.stream, s.tile_rows, s.tile_cols, s.slab_bytes) == (1, 256, 64, 64)
    s = nat.table_lookup(nat.PASS_FWD, torch.float32, 300000, 32, 64, 27)       # ... of fp32: 128-byte slabs as before
    assert (s.stream, s.tile_rows, s.tile_cols, s.slab_bytes) == (1, 256, 64, 128)
    s = nat.table_lookup(nat.PASS_FWD, torch.float16, 15192, 256, 256, 27)      # 119 tiles of 128 x 256: 64-column tiles instead
    assert (s.stream, s.tile_rows, s.tile_cols, s.slab_bytes) == (1, 256, 64, 128)
    s = nat.table_lookup(nat.PASS_FWD, torch.float16, 64160, 256, 256, 27)
    assert (s.stream, s.tile_rows, s.tile_cols, s.slab_bytes) == (1, 128, 256, 128)
    assert nat.table_lookup(nat.PASS_FWD, torch.float16, 5000, 192, 160, 27).stream == 0
    assert nat.table_lookup(nat.PASS_WGRAD, torch.float32, 300000, 192, 160, 27).stream == 0
    assert L.fgx_weight_panel_bytes(0, 0, 128, 128, 27, 64, 128) == 27 * 2 * 128 * 128
    assert L.fgx_weight_panel_bytes(2, 1, 40, 24, 27, 128, 32) == 27 * 1 * 64 * 128  # K=24 -> 1 slab, cols 40 -> 64
    assert L.fgx_weight_panel_bytes(2, 1, 40, 24, 27, 64, 32) == 27 * 2 * 64 * 64    # 16 floats per slab -> 2 slabs
    assert L.fgx_conv_scratch_bytes(ctypes.c_size_t(1000), 64, 1) == 0
    assert L.fgx_conv_scratch_bytes(ctypes.c_size_t(1000), 64, 4) == 4 * 1000 * 64 * 4
    # 1000 rows in blocks of 256 -> 4 blocks: bounds table (3 * 5 uint32, padded to 256 B) + 4 * 3 partial products
    # + the bias gradient's column sums per block and slice (4 blocks * 4 slices * Co floats) + the scratch of fgx_colsum
    colsum = L.fgx_colsum_scratch_bytes(ctypes.c_size_t(1000), 64)
    assert L.fgx_wgrad_scratch_bytes(ctypes.c_size_t(1000), 3, 48, 64, 256) == 256 + 4 * 3 * 48 * 64 * 4 + 4 * 4 * 64 * 4 + colsum
    # up to 32 channels on either side: room for the four partial products per block of the 32 x 32 streaming tile
    colsum = L.fgx_colsum_scratch_bytes(ctypes.c_size_t(1000), 16)
    assert L.fgx_wgrad_scratch_bytes(ctypes.c_size_t(1000), 3, 8, 16, 256) == 256 + 4 * 4 * 3 * 8 * 16 * 4 + 4 * 4 * 16 * 4 + colsum


def test_table_leaves_very_wide_layers_to_the_tiled_kernel(library):
    # the persistent gather GEMM stages the bias of all output columns in LDS beside its rings: from about 1900 columns
    # on that no longer fits, and the table must not pick it (any channel count has to run)
    import torch
    for c in (2048, 4096):
        for p in (nat.PASS_FWD, nat.PASS_DGRAD):
            s = nat.table_lookup(p, torch.float16, 100000, c, c, 27)
            assert s.stream == 0 and s.tile_cols == 128 and s.splitk >= 1, (c, p)
    assert nat.table_lookup(nat.PASS_FWD, torch.float16, 100000, 1024, 1920, 27).stream == 1
    assert nat.table_lookup(nat.PASS_FWD, torch.float16, 100000, 1024, 1921, 27).stream == 0
    assert nat.table_lookup(nat.PASS_DGRAD, torch.float16, 100000, 2048, 1024, 27).stream == 0   # dgrad: columns = Ci
    assert nat.table_lookup(nat.PASS_DGRAD, torch.float16, 100000, 1024, 2048, 27).stream == 1


def test_argument_errors_map_to_exceptions(library):
    L = nat.lib()
    with pytest.raises(ValueError):
        nat.check(L.fgx_hash_init(None, 16, ctypes.c_size_t(8), None))
    assert b"key_bits" in L.fgx_last_error()
    with pytest.raises(ValueError):
        nat.check(L.fgx_subm_neighbor_map(None, 32, None, ctypes.c_size_t(0), None, ctypes.c_size_t(0), 4, 4, 4,
                                          2, 3, 3, 1, 1, 1, None, None, None, None))
    with pytest.raises(ValueError):
        nat.check(L.fgx_conv_wgrad(0, None, None, None, None, None, None, ctypes.c_size_t(0), ctypes.c_size_t(0), 8, 8, 27, 128, 128, 0, 0,
                                   None, None, None, -1, None))
    with pytest.raises(ValueError):   # the streaming GEMM checks its arguments before touching the device
        nat.check(L.fgx_conv_gather_gemm_stream(0, None, None, None, None, None, None, None, None, ctypes.c_size_t(0),
                                                ctypes.c_size_t(10), ctypes.c_size_t(10), 128, 128, 27, 256, 128, 128, None, 0, None, None))
    assert b"null buffer" in L.fgx_last_error()
    with pytest.raises(ValueError):   # an activation code the kernels do not know
        nat.check(L.fgx_conv_gather_gemm_stream_act(0, None, None, None, None, None, None, None, None, ctypes.c_size_t(0),
                                                    ctypes.c_size_t(10), ctypes.c_size_t(10), 128, 128, 27, 256, 128, 128, None, 0,
                                                    7, None, None))
    assert b"activation" in L.fgx_last_error()
    with pytest.raises(ValueError):
        nat.check(L.fgx_conv_gather_gemm_act(0, None, None, None, None, None, None, ctypes.c_size_t(10), 128, 128, 27, 128, 128, 64, 1,
                                             None, 7, None, None))
    assert b"activation" in L.fgx_last_error()


def test_entry_points_of_the_resident_row_kernels_and_the_one_call_cache_check_their_arguments(library):
    L = nat.lib()
    sz = ctypes.c_size_t
    # sizes: pure functions of their arguments
    assert L.fgx_narrow_plan_bytes(sz(0), 27) == 256 and L.fgx_narrow_plan_bytes(sz(129), 27) == 256 + 2 * 10496
    assert L.fgx_narrow_plan_bytes(sz(128), 32) == 0                      # kernel volumes up to 31
    assert L.fgx_subm_cache_workspace_bytes(sz(1000), 32, 3, 3, 3, 1) >= L.fgx_subm_cache_workspace_bytes(sz(1000), 32, 3, 3, 3, 0) > 0
    assert L.fgx_subm_cache_workspace_bytes(sz(1000), 16, 3, 3, 3, 1) == 0 and L.fgx_subm_cache_workspace_bytes(sz(1000), 32, 3, 3, 5, 1) == 0
    with pytest.raises(ValueError):   # a kernel volume the mask codes cannot hold
        nat.check(L.fgx_subm_cache_build(None, sz(10), 1, 8, 8, 8, 3, 3, 5, 1, 1, 1, 32, 2, 0, None, sz(0), None, None, None, None,
                                         None, None, None, None))
    assert b"kernel volume" in L.fgx_last_error()
    with pytest.raises(ValueError):   # pair lists without a segment table
        nat.check(L.fgx_subm_cache_build(None, sz(10), 1, 8, 8, 8, 3, 3, 3, 1, 1, 1, 32, 2, 1, None, sz(0), None, None, None, None,
                                         None, None, None, None))
    assert b"segment table" in L.fgx_last_error()
    with pytest.raises(ValueError):
        nat.check(L.fgx_subm_cache_build(None, sz(10), 1, 8, 8, 8, 3, 3, 3, 1, 1, 1, 32, 2, 0, None, sz(0), None, None, None, None,
                                         None, None, None, None))
    assert b"null buffer" in L.fgx_last_error()
    with pytest.raises(ValueError):   # channel counts the resident-row GEMM does not take
        nat.check(L.fgx_conv_narrow_gemm(0, None, None, None, None, None, sz(10), sz(10), 48, 32, 27, 0, None, None, None))
    assert b"8, 16, 24 or 32" in L.fgx_last_error()
    with pytest.raises(ValueError):
        nat.check(L.fgx_conv_narrow_gemm(2, None, None, None, None, None, sz(10), sz(10), 32, 32, 27, 0, None, None, None))
    assert b"16-bit" in L.fgx_last_error()
    with pytest.raises(ValueError):
        nat.check(L.fgx_locality_order_grid(None, None, sz(10), 27, 8192, 17, 0, None, None, sz(0), None))
    assert b"bits per axis" in L.fgx_last_error()
    with pytest.raises(ValueError):
        nat.check(L.fgx_zorder_rows(None, sz(10), 16, 17, None, None, sz(0), None))
    assert b"64-bit key" in L.fgx_last_error()


def test_host_logic_without_gpu():
    import torch
    import flex_gemm
    from flex_gemm.ops.spconv import Algorithm, SubMConv3dFunction, SubMConv3dNeighborCache
    coords = torch.zeros((1, 4), dtype=torch.int32)
    flex_gemm.ops.spconv.set_algorithm(Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)
    with pytest.raises(NotImplementedError):
        SubMConv3dFunction._compute_neighbor_cache(coords, torch.Size([1, 1, 4, 4, 4]), (3, 3, 3), (1, 1, 1), False)
    with pytest.raises(AssertionError):
        SubMConv3dFunction._compute_neighbor_cache(coords.long(), torch.Size([1, 1, 4, 4, 4]), (3, 3, 3), (1, 1, 1), False)
    flex_gemm.ops.spconv.set_algorithm("nonsense")
    with pytest.raises(ValueError):
        SubMConv3dFunction._compute_neighbor_cache(coords, torch.Size([1, 1, 4, 4, 4]), (3, 3, 3), (1, 1, 1), False)
    flex_gemm.ops.spconv.set_algorithm(Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)
    c = SubMConv3dNeighborCache(a=1)
    c["b"] = 2
    assert c["a"] == 1 and c.b == 2
    with pytest.raises(AttributeError):
        c["missing"]
    # masked algorithms never fall back to the CPU
    with pytest.raises(NotImplementedError):
        SubMConv3dFunction._sparse_submanifold_conv_forward(
            torch.zeros(1, 8), SubMConv3dNeighborCache(neighbor_map=torch.zeros((1, 27), dtype=torch.int32)),
            torch.zeros(8, 3, 3, 3, 8), None)


def test_explicit_algorithm_matches_oracle_on_cpu():
    """The EXPLICIT_GEMM algorithm is plain torch ops and runs on any device, like the reference's."""
    import numpy as np
    import torch
    import flex_gemm
    from flex_gemm.ops.spconv import Algorithm, SubMConv3dFunction, sparse_submanifold_conv3d
    from flexgemm_amd.workloads import reference_test_shell
    from oracle import explicit_gemm as eg
    from oracle import neighbor as nb
    flex_gemm.ops.spconv.set_algorithm(Algorithm.EXPLICIT_GEMM)
    try:
        res, ci, co = 8, 6, 5
        coords = torch.from_numpy(reference_test_shell(res))
        shape = torch.Size([1, ci, res, res, res])
        cache = SubMConv3dFunction._compute_neighbor_cache_torch(coords, shape, (3, 3, 3), (1, 1, 1))
        ref_map = nb.neighbor_map(coords.numpy(), tuple(shape))
        assert cache.neighbor_map.dtype == torch.uint32
        assert np.array_equal(cache.neighbor_map.numpy(), ref_map)
        g = torch.Generator().manual_seed(0)
        feats = torch.randn(len(coords), ci, generator=g, dtype=torch.float64, requires_grad=True)
        weight = torch.randn(co, 3, 3, 3, ci, generator=g, dtype=torch.float64, requires_grad=True)
        bias = torch.randn(co, generator=g, dtype=torch.float64, requires_grad=True)
        out, cache2 = sparse_submanifold_conv3d(feats, coords, shape, weight, bias, neighbor_cache=cache)
        assert cache2 is cache
        grad = torch.randn(len(coords), co, generator=g, dtype=torch.float64)
        out.backward(grad)
        nm = torch.from_numpy(ref_map.view(np.int32))
        assert torch.allclose(out.detach(), eg.forward(feats.detach(), nm, weight.detach(), bias.detach()))
        gi, gw, gb = eg.backward(grad, feats.detach(), nm, weight.detach())
        assert torch.allclose(feats.grad, gi) and torch.allclose(weight.grad, gw) and torch.allclose(bias.grad, gb)
    finally:
        flex_gemm.ops.spconv.set_algorithm(Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)


def test_wgrad_block_rule_keeps_its_promises(library):
    """The schedule rule for wgrad's voxel blocks: whole kibi-rows, even blocks, never more fp32 partial products than the
    256 MiB cap allows; on the streaming kernel, the tile shape and block count that the balanced work lists were measured
    best with (the largest tile shape whose items fill the chip one and a half times, few blocks under many tiles)."""
    import torch
    for c in (32, 64, 128, 256, 512, 1024):
        for n in (1, 192, 848, 3840, 15192, 42608, 64160, 166232, 300000, 669288, 1026536, 2667120):
            s = nat.table_lookup(nat.PASS_WGRAD, torch.float16, n, c, c, 27)
            rows = s.block_rows
            assert rows >= 1024 and rows % 1024 == 0, (n, c, rows)
            if s.stream == 2:           # the sweep: block_rows is its sub-block size, it has no voxel blocks
                assert c in (64, 128) and n >= 8192, (n, c)
                continue
            blocks = -(-n // rows)
            slices = 4 if (s.stream and s.tile_rows == 32) else 1
            if blocks > 1:
                assert blocks * slices * 27 * c * c * 4 <= 256 << 20, (n, c, rows, "partial products exceed the cap")
                assert n - (blocks - 1) * rows > rows // 2 or blocks > 4, (n, c, rows, "short last block")
            # 16-bit types stream from 512 voxels on, under weights of 512 x 512 and more from 128 on
            assert s.stream == (1 if (n >= 512 or (n >= 128 and c >= 512)) else 0), (n, c)
            if s.stream == 1:
                tiles = -(-c // s.tile_rows) * -(-c // s.tile_cols)
                items = 27 * tiles * blocks
                assert items <= 4096 or n > 1 << 20, (n, c, "more items than the work lists take")
                # 256 x 128 tiles only from about three thousand voxels on and only where their items fill the chip
                if s.tile_rows == 256:
                    assert c >= 256 and n >= 3072 and items >= 384, (n, c, items)
                # few tiles: blocks of at most 16384 rows (an XCD's L2), unless the cap asks for longer ones
                if tiles <= 4 and rows > 16384:
                    assert -(-n // (rows - 1024)) > max((256 << 20) // (27 * c * c * 4 * slices), 1), (n, c, rows)
    expect = {(848, 256): (64, 64, 1024), (3840, 256): (64, 64, 4096), (15192, 256): (128, 128, 4096), (166232, 256): (256, 128, 15360),
              (3840, 512): (128, 128, 4096), (64160, 512): (256, 128, 21504), (42608, 1024): (256, 128, 43008), (848, 1024): (128, 128, 1024),
              (15192, 32): (32, 32, 2048), (64160, 32): (32, 32, 6144), (848, 128): (64, 64, 1024)}
    for (n, c), want in expect.items():
        s = nat.table_lookup(nat.PASS_WGRAD, torch.float16, n, c, c, 27)
        assert (s.tile_rows, s.tile_cols, s.block_rows, s.stream) == want + (1,), (n, c)
