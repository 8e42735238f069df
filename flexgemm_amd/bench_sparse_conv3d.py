#!/usr/bin/env python3
"""Timing of the generic sparse convolution (stride / padding) on one MI355X:  python -m flexgemm_amd.bench_sparse_conv3d

Input: the res-512 shell of the headline submanifold benchmark (669 288 voxels) with C channels, fp16.  For each
geometry it times, with HIP events, the output-coordinate builder, the neighbor-cache build, and one training step
(forward + input gradient + weight gradient + bias gradient) with the cache reused, and prints one JSON line per
geometry.  Effective TFLOP/s counts 2 * L * Ci * Co per pass, L = valid (output, kernel position) pairs, the same
accounting as the submanifold benchmark.
"""
from __future__ import annotations

import argparse
import json
import statistics

import torch

GEOMETRIES = {
    "k2s2": ((2, 2, 2), (2, 2, 2), (0, 0, 0), (1, 1, 1)),     # the downsampling layer of U-Net-style sparse networks
    "k3s2p1": ((3, 3, 3), (2, 2, 2), (1, 1, 1), (1, 1, 1)),
    "k3s1p1": ((3, 3, 3), (1, 1, 1), (1, 1, 1), (1, 1, 1)),   # output set = the input dilated by one voxel
}


def _time(fn, warmup, iters):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ms = []
    for _ in range(iters):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        torch.cuda.synchronize()
        ms.append(e0.elapsed_time(e1))
    return statistics.median(ms)


def main():
    p = argparse.ArgumentParser()
    p.add_argument("--res", type=int, default=512)
    p.add_argument("--channels", type=int, default=128)
    p.add_argument("--iters", type=int, default=20)
    p.add_argument("--warmup", type=int, default=3)
    p.add_argument("--geometry", default="all", choices=["all"] + list(GEOMETRIES))
    args = p.parse_args()

    import flex_gemm
    from flex_gemm.ops.spconv import Algorithm, SparseConv3dFunction
    from flexgemm_amd import _native as nat
    from flexgemm_amd.workloads import shell_coords

    assert torch.cuda.is_available(), "needs a GPU"
    nat.lib()
    dev = torch.device("cuda:0")
    flex_gemm.ops.spconv.set_algorithm(Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)
    res, c = args.res, args.channels
    coords = torch.from_numpy(shell_coords(res)).to(dev)
    shape = torch.Size([1, c, res, res, res])
    m = coords.shape[0]
    g = torch.Generator().manual_seed(0)
    feats = torch.randn(m, c, generator=g).half().to(dev).requires_grad_(True)
    weight_of = {}
    for name, (ks, st, pd, dl) in GEOMETRIES.items():
        if args.geometry not in ("all", name):
            continue
        v = ks[0] * ks[1] * ks[2]
        if ks not in weight_of:
            weight_of[ks] = (torch.randn(c, *ks, c, generator=g) / (v * c) ** 0.5).half().to(dev).requires_grad_(True)
        weight = weight_of[ks]
        bias = torch.randn(c, generator=g).half().to(dev).requires_grad_(True)
        oc = SparseConv3dFunction._get_output_coords(coords, shape, ks, st, pd, dl)
        t_coords = _time(lambda: SparseConv3dFunction._get_output_coords(coords, shape, ks, st, pd, dl), 1, 5)
        cache = SparseConv3dFunction._compute_neighbor_cache(coords, oc, shape, ks, st, pd, dl, True)
        t_cache = _time(lambda: SparseConv3dFunction._compute_neighbor_cache(coords, oc, shape, ks, st, pd, dl, True), 1, 5)
        pairs = int(cache._seg_host()[-1])
        grad = torch.randn(oc.shape[0], c, generator=g).half().to(dev)
        t_fwd = _time(lambda: SparseConv3dFunction._sparse_conv_forward(feats.detach(), cache, weight.detach(), bias.detach()),
                      args.warmup, args.iters)
        t_step = _time(lambda: (SparseConv3dFunction._sparse_conv_forward(feats.detach(), cache, weight.detach(), bias.detach()),
                                SparseConv3dFunction._sparse_conv_backward(grad, feats, cache, weight, bias)),
                       args.warmup, args.iters)
        flop = 2.0 * pairs * c * c
        print(json.dumps({
            "geometry": name, "kernel": ks, "stride": st, "padding": pd, "dilation": dl, "dtype": "f16", "channels": c,
            "n_in": m, "n_out": int(oc.shape[0]), "valid_pairs": pairs,
            "out_coords_ms": round(t_coords, 4), "neighbor_cache_ms": round(t_cache, 4),
            "forward_ms": round(t_fwd, 4), "train_step_ms": round(t_step, 4),
            "forward_tflops": round(flop / t_fwd / 1e9, 1), "train_step_tflops": round(3 * flop / t_step / 1e9, 1),
            "backward_mask_sorted": hasattr(cache, "sorted_idx_bwd"),
        }), flush=True)


if __name__ == "__main__":
    main()
