"""The entry point that allocates nothing: fgx_colsum_static keeps its partial sums in an array the library holds on the
GPU, and must give fgx_colsum's bits -- on two calls in a row, the second on a smaller input (the array then still
holds the first call's partial sums)."""
import ctypes as C
import sys

import pytest
import torch

from flexgemm_amd import _native as nat

pytestmark = pytest.mark.gpu


def _say(msg):
    print(f"[case] {msg}", flush=True)
    sys.stdout.flush()


def _colsum_pair(x):
    """(fgx_colsum with caller-owned scratch, fgx_colsum_static) on the same tensor"""
    L = nat.lib()
    n, cols = x.shape
    code = nat.DTYPE_CODE[x.dtype]
    want = torch.empty((cols,), dtype=x.dtype, device=x.device)
    got = torch.full((cols,), float("nan"), dtype=x.dtype, device=x.device)
    scratch = nat.workspace(L.fgx_colsum_scratch_bytes(nat.sz(n), C.c_int(cols)), x.device)
    with torch.cuda.device(x.device):
        nat.check(L.fgx_colsum(C.c_int(code), nat.ptr(x), nat.sz(n), C.c_int(cols), nat.ptr(scratch), nat.ptr(want), nat.stream()))
        nat.check(L.fgx_colsum_static(C.c_int(code), nat.ptr(x), nat.sz(n), C.c_int(cols), nat.ptr(got), nat.stream()))
    torch.cuda.synchronize()
    return want, got


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_static_scratch_colsum_equals_colsum_on_two_calls_in_a_row(gpu_device, dtype):
    g = torch.Generator().manual_seed(3)
    # first a large input that fills every slice of the partial sums, then smaller ones (fewer slices, fewer and odd
    # column counts) that must not see what the first left behind
    for n, cols in [(300000, 512), (5000, 128), (777, 40), (1, 2048), (0, 64)]:
        _say(f"colsum static n={n} cols={cols} {dtype}")
        x = torch.randn(n, cols, generator=g).to(dtype).to(gpu_device)
        want, got = _colsum_pair(x)
        assert torch.equal(want, got), f"n={n} cols={cols}: static-scratch result differs"
        if n:
            ref = x.double().sum(0)
            assert float((got.double() - ref).abs().max()) <= 1e-2 * max(float(ref.abs().max()), 1.0)
        else:
            assert (got == 0).all()


def test_static_scratch_colsum_rejects_what_does_not_fit(gpu_device):
    L = nat.lib()
    assert L.fgx_colsum_static_max_cols() == 2048
    x = torch.zeros((4, 2056), dtype=torch.float16, device=gpu_device)
    out = torch.empty((2056,), dtype=torch.float16, device=gpu_device)
    with pytest.raises(ValueError):
        nat.check(L.fgx_colsum_static(C.c_int(nat.DTYPE_CODE[x.dtype]), nat.ptr(x), nat.sz(4), C.c_int(2056), nat.ptr(out), nat.stream()))
    assert b"2048" in L.fgx_last_error()


def test_static_scratch_colsum_allocates_nothing_and_replays_in_a_graph(gpu_device):
    """After the per-device preparation a call leaves the allocator and the device's free memory alone, and it can be
    captured: every replay, with eager work and synchronisations in between, gives fgx_colsum's bits for the input the
    captured buffer holds at that moment."""
    L = nat.lib()
    dtype = torch.float16
    code = nat.DTYPE_CODE[dtype]
    g = torch.Generator().manual_seed(11)
    n, cols = 40000, 256
    x = torch.randn(n, cols, generator=g).to(dtype).to(gpu_device)
    out = torch.empty((cols,), dtype=dtype, device=gpu_device)
    with torch.cuda.device(gpu_device):
        nat.check(L.fgx_colsum_static_prepare())
        # one ordinary call first: the kernels are loaded, and the array holds old partial sums
        nat.check(L.fgx_colsum_static(C.c_int(code), nat.ptr(x), nat.sz(n), C.c_int(cols), nat.ptr(out), nat.stream()))
        torch.cuda.synchronize()
        _say("colsum static: allocation check")
        allocated, reserved = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
        free_before, _ = torch.cuda.mem_get_info()
        nat.check(L.fgx_colsum_static(C.c_int(code), nat.ptr(x), nat.sz(n), C.c_int(cols), nat.ptr(out), nat.stream()))
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info()
        assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == (allocated, reserved)
        assert free_after == free_before, "device memory changed across a call that must allocate nothing"

        _say("colsum static: capture")
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            nat.check(L.fgx_colsum_static(C.c_int(code), nat.ptr(x), nat.sz(n), C.c_int(cols), nat.ptr(out), nat.stream()))
        for replay in range(4):
            _say(f"colsum static: replay {replay}")
            fresh = torch.randn(n, cols, generator=g).to(dtype).to(gpu_device)
            x.copy_(fresh)
            out.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            want, eager = _colsum_pair(fresh)           # eager work between the replays
            assert torch.equal(out, want), f"replay {replay} differs from the eager result"
            assert torch.equal(eager, want)
