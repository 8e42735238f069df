#!/usr/bin/env python3
"""Training (or inference) time of L stacked submanifold convolutions on one MI355X:
    python -m flexgemm_amd.bench_train_stack [--mode train|inference]

The loop of the reference's training benchmark (tests/submconv/train_benchmark.py:152-160, configurations :165-174):
every iteration builds the neighbor cache for the coordinates, runs L layers `sparse_submanifold_conv3d(h, coords, shape,
weight_i, bias_i, neighbor_cache)` through autograd and calls backward with a tensor of ones.  The geometry is the
reference's test shell (tests/utils.py:6-25), dtype fp16, weights N(0,1) as there.  Everything goes through the public
operator, so Python, autograd and launch overheads are inside the timed region, and the cache is built once per
iteration and shared by the L layers.  --mode inference is the loop of the reference's inference benchmark
(tests/submconv/inf_benchmark.py:149-157, same configurations): the cache is built without the gradient tables and only
the L forward passes run (autograd still records them, as there: the weights are parameters).

Prints one JSON line per configuration: wall ms per iteration (median of HIP-event timings), the part of it spent in the
cache build, and effective TFLOP/s over 6 * pairs * C * C * L useful FLOP (forward + both gradients of every layer).
"""
from __future__ import annotations

import argparse
import json
import statistics

import torch

# (RES, C, L) of the reference's sweep, including the two it leaves commented out
CONFIGS = [(8, 1024, 16), (16, 1024, 8), (32, 1024, 4), (64, 1024, 2), (128, 512, 2), (256, 256, 2), (512, 128, 2), (1024, 64, 2)]


def _median_ms(fn, warmup, iters):
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
    p.add_argument("--iters", type=int, default=10)
    p.add_argument("--warmup", type=int, default=3)
    p.add_argument("--max-res", type=int, default=512, help="skip configurations above this resolution")
    p.add_argument("--mode", choices=("train", "inference"), default="train")
    p.add_argument("--graph", action="store_true",
                   help="the L forward passes (and, in train mode, the backward pass) are captured once into a HIP graph "
                        "and replayed (the neighbor cache is built once, outside the timed loop: a graph is tied to its "
                        "cache's tables)")
    p.add_argument("--panel-cache", action="store_true",
                   help="keep the repacked weight panels with the weights (flex_gemm.ops.spconv.set_weight_panel_cache): "
                        "the loop never updates its weights, so every pack after the second iteration is saved")
    p.add_argument("--relu", choices=("none", "fused", "fused-no-bits", "separate"), default="none",
                   help="a ReLU after every layer: in the GEMM's epilogue (sparse_submanifold_conv3d_relu; fused-no-bits: "
                        "its backward tests the saved output instead of the epilogue's bit mask) or as torch.relu")
    p.add_argument("--config", default="", help="RES,C,L: one configuration of its own instead of the reference's list")
    p.add_argument("--narrow", choices=("auto", "on", "off"), default="auto",
                   help="the resident-row kernels of narrow layers (flexgemm_amd.ops.spconv.NARROW_RESIDENT)")
    args = p.parse_args()

    import flex_gemm
    from flex_gemm.ops.spconv import Algorithm, SubMConv3dFunction, sparse_submanifold_conv3d, sparse_submanifold_conv3d_relu
    from flexgemm_amd.ops import spconv as spconv_config
    spconv_config.RELU_BIT_MASK = args.relu != "fused-no-bits"
    spconv_config.NARROW_RESIDENT = args.narrow
    configs = CONFIGS
    if args.config:
        configs = [tuple(int(x) for x in args.config.split(","))]
        args.max_res = max(args.max_res, configs[0][0])

    def layer(h, coords, shape, w, b, cache):
        if args.relu in ("fused", "fused-no-bits"):
            return sparse_submanifold_conv3d_relu(h, coords, shape, w, b, cache)[0]
        h = sparse_submanifold_conv3d(h, coords, shape, w, b, cache)[0]
        return torch.relu(h) if args.relu == "separate" else h
    from flexgemm_amd import _native as nat
    from flexgemm_amd.workloads import reference_test_shell

    assert torch.cuda.is_available(), "needs a GPU"
    nat.lib()
    dev = torch.device("cuda:0")
    flex_gemm.ops.spconv.set_algorithm(Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)
    flex_gemm.ops.spconv.set_weight_panel_cache(args.panel_cache, max_bytes=16 << 30)
    for res, c, layers in configs:
        if res > args.max_res:
            continue
        coords = torch.from_numpy(reference_test_shell(res)).to(dev)
        n = coords.shape[0]
        shape = torch.Size([1, c, res, res, res])
        g = torch.Generator().manual_seed(res)
        feats = torch.randn(n, c, generator=g).half().to(dev)
        params = [(torch.nn.Parameter(torch.randn(c, 3, 3, 3, c, generator=g).half().to(dev)),
                   torch.nn.Parameter(torch.randn(c, generator=g).half().to(dev))) for _ in range(layers)]

        train = args.mode == "train"

        def iteration():
            for w, b in params:
                w.grad = None
                b.grad = None
            cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), train)
            h = feats
            for w, b in params:
                h = layer(h, coords, shape, w, b, cache)
            if train:
                h.backward(torch.ones_like(h))

        def build_only():
            SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), train)

        if args.graph:
            fixed = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), train)
            ones = torch.ones((n, c), dtype=feats.dtype, device=dev)

            def whole_step():
                h = feats
                for w, b in params:
                    h = layer(h, coords, shape, w, b, fixed)
                if train:
                    h.backward(ones)
                return h

            with torch.set_grad_enabled(train):
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    for _ in range(3):
                        for w, b in params:
                            w.grad = None
                            b.grad = None
                        whole_step()
                torch.cuda.current_stream().wait_stream(side)
                torch.cuda.synchronize()
                for w, b in params:
                    w.grad = None              # the captured backward allocates the gradients in the graph's pool
                    b.grad = None
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    whole_step()
            iteration = graph.replay
        ms = _median_ms(iteration, args.warmup, args.iters)
        ms_build = _median_ms(build_only, 1, args.iters)
        cache = SubMConv3dFunction._compute_neighbor_cache(coords, shape, (3, 3, 3), (1, 1, 1), True)
        pairs = int(cache._seg_host()[-1])
        # the first layer's input needs no gradient: its dgrad pass is skipped, as in the reference
        passes = 3 * layers - 1 if train else layers
        flop = 2.0 * pairs * c * c * passes
        print(json.dumps({
            "benchmark": "L stacked submanifold 3x3x3 convolutions, " + ("forward + backward" if train else "forward only")
                         + (", replayed from a HIP graph, cache built once" if args.graph else ", cache built per iteration"),
            "weight_panel_cache": bool(args.panel_cache), "relu": args.relu, "res": res, "channels": c, "layers": layers, "voxels": n, "pairs": pairs, "dtype": "f16",
            "ms_per_iteration": round(ms, 4), "cache_build_ms": round(ms_build, 4), "gemm_passes": passes,
            "tflops": round(flop / (ms * 1e-3) / 1e12, 1),
        }), flush=True)


if __name__ == "__main__":
    main()
