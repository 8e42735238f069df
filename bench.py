#!/usr/bin/env python3
"""Benchmark of the submanifold sparse-conv hot path on one MI355X.

One "step" is one training pass of a single 3x3x3 submanifold conv layer over one synthetic batch:
forward + dgrad + wgrad (+ dbias) through the masked implicit GEMM, with the neighbor cache built once
before the timed region and reused (the reference's benchmark does the same: tests/submconv/train_benchmark.py:152-160).
Inputs are resident in HBM when the timed region starts.

Headline workload (N = 1): configuration 3 -- res 512 shell (669 288 voxels), Ci = Co = 128, fp16.
`value` = effective TFLOP/s = useful FLOP / time with useful FLOP = 6 * L * Ci * Co per step
(L = valid neighbor pairs; the reference's accounting: tests/submconv/fwd.py:247-249, bwd.py:288-290).

Prints ONE JSON line.  `--workload cfg2|cfg3|cfg4|cfg5` selects another configuration (cfg2 is forward only),
`--dtype f32` the fp32-input variant of a configuration (configuration 5 names one).

Timing follows the reference's protocol (tests/utils.py:35-65: events around every call, peak memory): besides the
wall-clock mean over the timed steps, the line carries median and minimum per step and per pass from HIP events,
the peak of allocated device memory over the timed region, and the neighbor-cache build split into its phases.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"f16": 2500.0, "bf16": 2500.0, "f32": 157.3}   # MI355X dense MFMA peaks
HBM_PEAK_GBS = 8000.0
# HBM-side bytes per launch of the dominant kernels come from two rocprofv3 counter runs of this script (FETCH_SIZE, then
# WRITE_SIZE, each scaled by what the same counter reads for the plain copy of --calibrate-copy), MFMA-busy share, clock and
# L2 hit rate from two more.  The counters cannot be read from inside the process: `python -m flexgemm_amd.profile_traffic`
# turns the counter files into an entry of this file, stamped with a digest of each kernel's source files, and the summary
# under profiles/ quotes the same entry.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def measured_counters(workload: str, dname: str, role: str):
    """{traffic_bytes, mfma_busy_frac, l2_hit, clock_ghz} per launch of a role's kernel ("gemm": the gather GEMM, "wgrad":
    the weight gradient) from profiles/traffic.json; every value is None when there is no entry for this workload and
    dtype or the kernel's sources have changed since it was measured."""
    from flexgemm_amd.profile_traffic import source_digest
    keys = ("traffic_bytes", "mfma_busy_frac", "l2_hit", "clock_ghz")
    none = {k: None for k in keys}
    try:
        with open(TRAFFIC_FILE) as f:
            entry = json.load(f).get(f"{workload}_{dname}", {}).get(role)
    except (OSError, ValueError):
        return none
    if not entry or entry.get("source_digest") != source_digest(entry.get("sources", [])):
        return none
    return {k: entry.get(k) for k in keys}


def _finite(obj):
    """The same structure with NaN and infinities replaced by None (they are not JSON)."""
    if isinstance(obj, float):
        return obj if math.isfinite(obj) else None
    if isinstance(obj, dict):
        return {k: _finite(v) for k, v in obj.items()}
    if isinstance(obj, (list, tuple)):
        return [_finite(v) for v in obj]
    return obj


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=50)
    p.add_argument("--warmup", type=int, default=5)
    p.add_argument("--workload", default="cfg3", choices=["cfg2", "cfg3", "cfg4", "cfg5"])
    p.add_argument("--dtype", default=None, choices=["f16", "bf16", "f32"], help="override the configuration's dtype")
    p.add_argument("--wgrad-sweep", type=int, default=0, metavar="SUB_ROWS",
                   help="run wgrad as the sweep (fgx_conv_wgrad_sweep) with sub-blocks of SUB_ROWS voxels instead of the table's schedule")
    p.add_argument("--wgrad-sweep-lead", type=int, default=3, help="sub-blocks a workgroup may run ahead when paced")
    p.add_argument("--wgrad-sweep-polls", type=int, default=0, help="poll limit of the sweep's pacing, 0 = unpaced")
    p.add_argument("--wgrad-block-major", type=int, default=0, metavar="BLOCK_ROWS",
                   help="run wgrad with the block-major streaming kernel (fgx_conv_wgrad) on voxel blocks of BLOCK_ROWS rows instead of the table's schedule")
    p.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU leg (used under rocprofv3)")
    p.add_argument("--cpu-rows", type=int, default=0, help="rows in the CPU baseline sample (0 = auto)")
    p.add_argument("--build-only", action="store_true", help="time only the neighbor-cache build")
    p.add_argument("--no-others", action="store_true", help="skip the other configurations that follow the headline one")
    p.add_argument("--other-steps", type=int, default=30, help="timed steps of each of the other configurations (after 5 warm-up steps)")
    p.add_argument("--calibrate-copy", action="store_true",
                   help="also run a plain 1 GiB device copy (reference point for FETCH_SIZE / WRITE_SIZE counters)")
    return p.parse_args()


def cpu_baseline(wl, nmap_cpu, passes, rows_hint):
    """Explicit gather-GEMM oracle (torch CPU, fp32) timed on a bounded row sample of the same workload."""
    import torch
    from oracle import explicit_gemm as eg
    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    c = wl.channels
    rows = rows_hint or max(1024, min(wl.n, int(3.0e8 / (27 * c))))     # im2col sample <= 0.3 G elements
    rows = min(rows, wl.n)
    sel = torch.arange(rows)
    sub = nmap_cpu[sel]
    f32, w32, b32, g32 = wl.feats.float(), wl.weight.float(), wl.bias.float(), wl.grad.float()
    l_sample = int((sub >= 0).sum())

    def run():
        eg.forward(f32, sub, w32, b32)
        if passes == 3:
            # dgrad for the sampled output rows; wgrad contribution of the sampled rows; dbias of the sample
            inv = torch.flip(sub.long(), [1])
            wt = w32.reshape(c, 27, c).transpose(0, 1).reshape(27 * c, c)
            torch.mm(eg._im2col(g32, inv), wt)
            torch.mm(eg._im2col(f32, sub.long()).t(), g32[sel])
            g32[sel].sum(0)

    run()                                   # warm-up (page faults, thread pool)
    t0 = time.perf_counter()
    iters = 0
    while True:
        run()
        iters += 1
        if time.perf_counter() - t0 > 10.0 or iters >= 20:
            break
    dt = (time.perf_counter() - t0) / iters
    flop = 2.0 * l_sample * c * c * passes
    return {
        "value": flop / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": f"first {rows} rows of {wl.name} ({l_sample} valid pairs), {'fwd+dgrad+wgrad' if passes == 3 else 'fwd'}, "
                  f"explicit gather-GEMM in torch CPU fp32 (substituted for {str(wl.dtype).split('.')[-1]}), {iters} iters, "
                  f"{dt * 1e3:.1f} ms/iter",
    }


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the hot path is a single-device operator); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    import flex_gemm
    from flex_gemm.ops.spconv import Algorithm, SubMConv3dFunction
    from flexgemm_amd import _native as nat
    from flexgemm_amd.workloads import make_workload

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    nat.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    flex_gemm.ops.spconv.set_algorithm(Algorithm.MASKED_IMPLICIT_GEMM_SPLITK)

    names = {torch.float16: "f16", torch.bfloat16: "bf16", torch.float32: "f32"}
    from flexgemm_amd.ops.spconv import submanifold_conv3d as impl
    impl.WGRAD_SWEEP_LEAD, impl.WGRAD_SWEEP_MAX_POLLS = args.wgrad_sweep_lead, args.wgrad_sweep_polls
    if args.wgrad_sweep or args.wgrad_block_major:
        table = nat.table_lookup

        def with_wgrad_kernel(pass_kind, *a):
            sc = table(pass_kind, *a)
            if pass_kind == nat.PASS_WGRAD:
                if args.wgrad_sweep:
                    sc.stream, sc.block_rows = 2, args.wgrad_sweep
                else:
                    sc.stream, sc.block_rows = 1, args.wgrad_block_major
            return sc
        nat.table_lookup = with_wgrad_kernel

    def measure(workload, dtype_name, steps, warmup, full, time_hash_builder=False):
        """One configuration: cache build (timed), warm-up, `steps` timed steps.  full: also the build's phases."""
        wl = make_workload(workload, dtype={v: k for k, v in names.items()}.get(dtype_name))
        dt = wl.dtype
        dname = names[dt]
        c = wl.channels
        passes = 1 if workload == "cfg2" else 3
        coords = wl.coords.to(dev)
        feats = wl.feats.to(dt).to(dev).requires_grad_(passes == 3)
        weight = wl.weight.to(dt).to(dev).requires_grad_(passes == 3)
        bias = wl.bias.to(dt).to(dev).requires_grad_(passes == 3)
        grad = wl.grad.to(dt).to(dev)

        # ---- neighbor cache: built once, timed separately ----
        def build_cache():
            return SubMConv3dFunction._compute_neighbor_cache(coords, wl.shape, (3, 3, 3), (1, 1, 1), passes == 3)

        cache = build_cache()
        torch.cuda.synchronize()
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        build_ms = []
        for _ in range(5):
            ev0.record()
            cache = build_cache()
            ev1.record()
            torch.cuda.synchronize()
            build_ms.append(ev0.elapsed_time(ev1))
        build_ms.sort()
        hash_build_ms = None
        if time_hash_builder:
            flex_gemm.ops.spconv.set_neighbor_map_builder("hash")
            try:
                hash_build_ms = []
                for _ in range(4):          # (the first one also warms the allocator up for the hash table)
                    ev0.record()
                    build_cache()
                    ev1.record()
                    torch.cuda.synchronize()
                    hash_build_ms.append(ev0.elapsed_time(ev1))
                hash_build_ms = sorted(hash_build_ms[1:])
            finally:
                flex_gemm.ops.spconv.set_neighbor_map_builder("auto")

        # the build split into its phases: the library names them to a hook, which records an event on their stream; the
        # first forward of a fresh cache adds the tables made on first use (tile masks, gather plan)
        def build_phases(reps=5):
            marks = []

            def hook(name, stream):
                # (the stream the library enqueues the phase on: the caller's, or the library's second one)
                e = torch.cuda.Event(enable_timing=True)
                on = torch.cuda.ExternalStream(stream) if stream else torch.cuda.current_stream()
                e.record(on)
                marks.append((name, e, on.cuda_stream))

            gap = "between calls (host: allocations, read-backs)"
            runs = []
            nat.set_phase_hook(hook)
            try:
                for _ in range(reps):
                    del marks[:]
                    fresh = build_cache()
                    with torch.no_grad():
                        SubMConv3dFunction._sparse_submanifold_conv_forward(feats, fresh, weight, bias)
                    torch.cuda.synchronize()
                    once = {}
                    # a phase lasts until the next mark on its own stream (the pair lists of a training cache are made
                    # on a second stream, beside the mask sort)
                    for sid in {m[2] for m in marks}:
                        mine = [m for m in marks if m[2] == sid]
                        for (name, e0, _), (_, e1, _) in zip(mine[:-1], mine[1:]):
                            once[name or gap] = once.get(name or gap, 0.0) + e0.elapsed_time(e1)
                    runs.append(once)
            finally:
                nat.set_phase_hook(None)
            return {k: sorted(r.get(k, 0.0) for r in runs)[len(runs) // 2] for k in runs[-1]}

        phases_ms = build_phases() if full else None
        pairs = int(cache.valid_signal_seg.view(torch.int32)[-1].item()) if passes == 3 else \
            int((cache.neighbor_map.view(torch.int32) != -1).sum().item())
        n = wl.n
        build_bytes = 152.0 * n + (8.0 * pairs + 4 * 28 if passes == 3 else 0.0)
        if args.build_only:
            return {"metric": "neighbor-cache build", "workload": workload, "n": n, "pairs": pairs,
                    "build_ms_median": build_ms[len(build_ms) // 2], "build_ms_min": build_ms[0],
                    "algorithmic_GBps": build_bytes / (build_ms[len(build_ms) // 2] * 1e-3) / 1e9,
                    "phases_ms_median": phases_ms}, None, None, None

        # ---- the step ----
        def step():
            out = SubMConv3dFunction._sparse_submanifold_conv_forward(feats, cache, weight, bias)
            if passes == 3:
                return out, SubMConv3dFunction._sparse_submanifold_conv_backward(grad, feats, cache, weight, bias)
            return out, None

        for _ in range(max(warmup, 1)):
            step()
        torch.cuda.synchronize()
        if args.calibrate_copy and full:
            # a plain copy kernel of known size: reads 1 GiB, writes 1 GiB per launch
            a = torch.empty(1 << 29, dtype=torch.float16, device=dev).fill_(1.0)
            b = torch.empty_like(a)
            for _ in range(3):
                torch.neg(a, out=b)
            torch.cuda.synchronize()
            del a, b

        # HIP events around the dominant kernel's launches, on the stream they are launched on
        events = {}

        def hook(name, phase):
            e = torch.cuda.Event(enable_timing=True)
            e.record(torch.cuda.current_stream())
            events.setdefault(name, []).append(e)

        nat.EVENT_HOOK = hook
        step_events = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats(dev)
        t0 = time.perf_counter()
        for i in range(steps):
            step_events[i].record()
            step()
        step_events[steps].record()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        nat.EVENT_HOOK = None
        peak_bytes = torch.cuda.max_memory_allocated(dev)

        ms_per_step = elapsed * 1e3 / steps
        step_ms = sorted(step_events[i].elapsed_time(step_events[i + 1]) for i in range(steps))
        flop_pass = 2.0 * pairs * c * c
        value = flop_pass * passes / (ms_per_step * 1e-3) / 1e12

        def pass_ms(names):
            """(mean, median, min, count) of the event-timed calls of these names"""
            ts = []
            for nm in names:
                ev = events.get(nm, [])
                ts += [ev[i].elapsed_time(ev[i + 1]) for i in range(0, len(ev) - 1, 2)]
            ts.sort()
            if not ts:
                return float("nan"), float("nan"), float("nan"), 0
            return sum(ts) / len(ts), ts[len(ts) // 2], ts[0], len(ts)

        def stats(names):
            mean, med, lo, cnt = pass_ms(names)
            return {"mean": mean, "median": med, "min": lo, "calls": cnt} if cnt else None

        gemm_ms, _, _, gemm_launches = pass_ms(["gather_gemm_fwd", "gather_gemm_dgrad"])
        wgrad_ms = pass_ms(["wgrad"])[0]
        es = 2 if dname != "f32" else 4
        gemm_bytes = es * n * (c + c) + es * 27 * c * c + 108.0 * n + 8.0 * n
        roof = {
            "bound": "mfma", "kernel": "gather GEMM (gather_gemm_stream_kernel or gather_gemm_kernel; forward and dgrad launches)",
            "achieved": flop_pass / (gemm_ms * 1e-3) / 1e12, "peak": PEAK_TFLOPS[dname], "unit": "TFLOP/s",
            "frac": flop_pass / (gemm_ms * 1e-3) / 1e12 / PEAK_TFLOPS[dname],
            "avg_launch_ms": gemm_ms, "launches_timed": gemm_launches,
            "algorithmic_flop_per_launch": flop_pass,
            "algorithmic_bytes_per_launch": gemm_bytes,
            "algorithmic_hbm_GBps": gemm_bytes / (gemm_ms * 1e-3) / 1e9,
        }
        seen = measured_counters(workload, dname, "gemm")
        roof.update({"traffic": seen["traffic_bytes"], "mfma_busy_frac": seen["mfma_busy_frac"], "l2_hit": seen["l2_hit"],
                     "clock_ghz": seen["clock_ghz"]})
        if c * es <= 64:   # rows of 64 bytes (configuration 4, C = 32): every pass is HBM bound
            roof.update({"bound": "hbm", "achieved": gemm_bytes / (gemm_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": gemm_bytes / (gemm_ms * 1e-3) / 1e9 / HBM_PEAK_GBS})

        wgrad_roof = None
        if passes == 3 and wgrad_ms == wgrad_ms:
            wgrad_bytes = es * n * (c + c) + 8.0 * pairs + es * 27 * c * c
            seen = measured_counters(workload, dname, "wgrad")
            wgrad_roof = {
                "bound": "mfma", "kernel": "weight gradient (wgrad_sweep_kernel + its reduction, or the block-major kernels)",
                "achieved": flop_pass / (wgrad_ms * 1e-3) / 1e12, "peak": PEAK_TFLOPS[dname], "unit": "TFLOP/s",
                "frac": flop_pass / (wgrad_ms * 1e-3) / 1e12 / PEAK_TFLOPS[dname], "avg_launch_ms": wgrad_ms,
                "algorithmic_flop_per_launch": flop_pass, "algorithmic_bytes_per_launch": wgrad_bytes,
                "traffic": seen["traffic_bytes"], "mfma_busy_frac": seen["mfma_busy_frac"], "l2_hit": seen["l2_hit"],
                "clock_ghz": seen["clock_ghz"]}
            if c * es <= 64:
                wgrad_roof.update({"bound": "hbm", "achieved": wgrad_bytes / (wgrad_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS,
                                   "unit": "GB/s", "frac": wgrad_bytes / (wgrad_ms * 1e-3) / 1e9 / HBM_PEAK_GBS})

        result = {
            "metric": "effective TFLOPS (useful MACs over valid neighbor pairs), submconv3d 3^3 "
                      + ("fwd+dgrad+wgrad" if passes == 3 else "fwd") + f", res{wl.res} C={c}",
            "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
            "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": dname, "data": "synthetic",
            "config": {"workload": f"{workload}: res {wl.res} shell, N={n}, L={pairs}, Ci=Co={c}, {dname}, "
                                   + ("fwd+dgrad+wgrad+dbias, neighbor cache prebuilt and reused" if passes == 3 else "forward"),
                       "n_voxels": n, "valid_pairs": pairs, "useful_gflop_per_step": flop_pass * passes / 1e9},
            "frac_of_mfma_peak": value / PEAK_TFLOPS[dname],
            "pass_ms": {"gather_gemm_avg": gemm_ms, "wgrad_incl_reduce": wgrad_ms if wgrad_ms == wgrad_ms else None,
                        "forward": stats(["gather_gemm_fwd"]), "dgrad": stats(["gather_gemm_dgrad"]), "wgrad": stats(["wgrad"])},
            "step_ms": {"wall_mean": ms_per_step, "median": step_ms[len(step_ms) // 2], "min": step_ms[0]},
            "peak_memory_bytes": peak_bytes,
            "neighbor_cache_build": {"ms_median": build_ms[len(build_ms) // 2], "ms_min": build_ms[0],
                                     "algorithmic_bytes": build_bytes,
                                     "algorithmic_GBps": build_bytes / (build_ms[len(build_ms) // 2] * 1e-3) / 1e9,
                                     "frac_of_hbm_peak": build_bytes / (build_ms[len(build_ms) // 2] * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                     "phases_ms_median": phases_ms},
            "roofline": roof,
            "wgrad_roofline": wgrad_roof,
        }
        if hash_build_ms:
            med = hash_build_ms[len(hash_build_ms) // 2]
            result["neighbor_cache_build"]["hash_builder"] = {
                "ms_median": med, "ms_min": hash_build_ms[0], "algorithmic_GBps": build_bytes / (med * 1e-3) / 1e9,
                "frac_of_hbm_peak": build_bytes / (med * 1e-3) / 1e9 / HBM_PEAK_GBS}
        return result, wl, cache, passes

    result, wl, cache, passes = measure(args.workload, args.dtype, args.steps, args.warmup, True)
    if args.build_only:
        print(json.dumps(_finite(result), allow_nan=False))
        return
    if not args.no_others and args.workload == "cfg3" and args.dtype is None:
        # the other configurations, a few steps each (no CPU leg, no phase split); configuration 4 also with the hash builder
        others = []
        for wname, dn in (("cfg2", None), ("cfg4", None), ("cfg5", None), ("cfg5", "f32")):
            try:
                r, _, _, _ = measure(wname, dn, args.other_steps, 5, False, time_hash_builder=(wname == "cfg4"))
            except Exception as exc:       # the headline line must come out whatever happens to a side measurement
                others.append({"workload": wname, "dtype": dn, "error": f"{type(exc).__name__}: {exc}"})
                torch.cuda.empty_cache()
                continue
            others.append({"workload": wname, "dtype": r["dtype"], "ms_per_step": r["ms_per_step"], "value": r["value"],
                           "unit": r["unit"], "steps": args.other_steps, "config": r["config"]["workload"],
                           "frac_of_mfma_peak": r["frac_of_mfma_peak"],
                           "roofline": {k: r["roofline"][k] for k in ("bound", "achieved", "peak", "unit", "frac", "avg_launch_ms")},
                           "wgrad_roofline": None if r["wgrad_roofline"] is None else
                           {k: r["wgrad_roofline"][k] for k in ("bound", "achieved", "peak", "unit", "frac", "avg_launch_ms")},
                           "pass_ms": r["pass_ms"], "step_ms": r["step_ms"],
                           "neighbor_cache_build": {k: v for k, v in r["neighbor_cache_build"].items() if k != "phases_ms_median"}})
            torch.cuda.empty_cache()
        result["other_workloads"] = others
    if not args.no_cpu_baseline:
        nmap_cpu = cache.neighbor_map.cpu().view(torch.int32)
        try:
            result["cpu_baseline"] = cpu_baseline(wl, nmap_cpu, passes, args.cpu_rows)
        except Exception as exc:           # (as above: never at the price of the line itself)
            result["cpu_baseline"] = {"error": f"{type(exc).__name__}: {exc}"}
    else:
        result["cpu_baseline"] = None
    print(json.dumps(_finite(result), allow_nan=False))


if __name__ == "__main__":
    main()
