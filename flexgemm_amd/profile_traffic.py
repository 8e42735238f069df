"""Counter figures per launch of the step's two dominant kernels from `rocprofv3 --pmc` runs of bench.py, kept in
profiles/traffic.json and printed as the table that the summary under profiles/ quotes.

rocprofv3 collects one counter set per run, so the figures come from four runs of the same command (each a few seconds):

    rocprofv3 --pmc FETCH_SIZE --output-format csv -d OUT/fetch -- python3 bench.py --steps 5 --warmup 2 --no-cpu-baseline --no-others --calibrate-copy
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d OUT/write -- python3 bench.py ... (same)
    rocprofv3 --pmc SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_VALU_MFMA_MOPS_F16 SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_WAIT_INST_ANY SQ_LDS_IDX_ACTIVE SQ_LDS_BANK_CONFLICT GRBM_GUI_ACTIVE --output-format csv -d OUT/sq -- python3 bench.py ... (same)
    rocprofv3 --pmc TCC_HIT_sum TCC_MISS_sum --output-format csv -d OUT/l2 -- python3 bench.py ... (same)

    python -m flexgemm_amd.profile_traffic --workload cfg3 --dtype f16 --fetch OUT/fetch --write OUT/write --sq OUT/sq --l2 OUT/l2

What is derived, per kernel (means over the dispatches of the run):

* fetch / write / traffic bytes: FETCH_SIZE and WRITE_SIZE (KiB per dispatch) scaled by what the same counter reads for
  the plain copy that `bench.py --calibrate-copy` adds (1 GiB read, 1 GiB written per launch);
* clock_ghz: GRBM_GUI_ACTIVE is summed over the 8 XCDs; divided by 8 and by the dispatch's duration (End_Timestamp -
  Start_Timestamp of the same CSV row) it is the clock the kernel ran at;
* mfma_busy_frac: SQ_VALU_MFMA_BUSY_CYCLES over (1024 SIMDs x the dispatch's cycles, GRBM_GUI_ACTIVE / 8) -- the share of
  the launch during which a SIMD's matrix pipe was busy, padded work included;
* l2_hit: TCC_HIT_sum / (TCC_HIT_sum + TCC_MISS_sum).

The entry "<workload>_<dtype>" carries, per role ("gemm": the streaming gather GEMM of forward and dgrad, "wgrad": the
sweep), these figures and a digest of the role's source files; bench.py reports them only while the digest still matches
the sources it runs.
"""
from __future__ import annotations

import argparse
import csv
import glob
import hashlib
import json
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")
COPY_BYTES = float(1 << 30)          # read and written per launch of the calibration copy
SIMDS = 256 * 4
XCDS = 8
# the sources each role's kernels are built from
ROLE_SOURCES = {
    "gemm": ["flexgemm_amd/csrc/conv_gemm_stream.hip", "flexgemm_amd/csrc/conv_gemm.hip", "flexgemm_amd/csrc/gemm_device.h",
             "flexgemm_amd/csrc/fgx_common.h", "flexgemm_amd/csrc/tuning.hip"],
    "wgrad": ["flexgemm_amd/csrc/wgrad_sweep.hip", "flexgemm_amd/csrc/wgrad_gemm.hip", "flexgemm_amd/csrc/wgrad_device.h",
              "flexgemm_amd/csrc/gemm_device.h", "flexgemm_amd/csrc/fgx_common.h", "flexgemm_amd/csrc/tuning.hip"],
}
GEMM_SOURCES = ROLE_SOURCES["gemm"]
ROLE_KERNEL = {"gemm": "gather_gemm_stream_kernel", "wgrad": "wgrad_sweep_kernel"}


def source_digest(paths) -> str:
    """sha256 (first 16 hex digits) over the named files, repository-relative, in the order given."""
    h = hashlib.sha256()
    for rel in paths:
        try:
            with open(os.path.join(ROOT, rel), "rb") as f:
                h.update(rel.encode() + b"\0" + f.read())
        except OSError:
            h.update(rel.encode() + b"\0<missing>")
    return h.hexdigest()[:16]


def short_name(kernel: str) -> str:
    k = re.sub(r"\(anonymous namespace\)::", "", kernel)
    k = re.sub(r"^void ", "", k)
    k = re.sub(r"\(.*$", "", k)
    return k.replace("fgx::", "")


def per_kernel(directory: str):
    """{short kernel name: {counter: mean value, "_us": mean duration, "_n": dispatches}} over every
    *_counter_collection.csv below `directory`."""
    acc = {}
    for path in glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True):
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                name = short_name(row["Kernel_Name"])
                slot = acc.setdefault(name, {})
                cnt, tot, dur = slot.get(row["Counter_Name"], (0, 0.0, 0.0))
                us = (int(row["End_Timestamp"]) - int(row["Start_Timestamp"])) / 1000.0
                slot[row["Counter_Name"]] = (cnt + 1, tot + float(row["Counter_Value"]), dur + us)
    out = {}
    for name, slot in acc.items():
        rec = {}
        for counter, (cnt, tot, dur) in slot.items():
            rec[counter] = tot / cnt
            rec["_us"] = dur / cnt
            rec["_n"] = cnt
        out[name] = rec
    return out


def per_kernel_mean(directory: str, counter: str):
    """{short kernel name: (dispatches, mean counter value)}"""
    return {k: (v["_n"], v[counter]) for k, v in per_kernel(directory).items() if counter in v}


def the_kernel(table, needle: str):
    hits = [k for k in table if needle in k]
    if len(hits) != 1:
        raise SystemExit(f"kernel {needle!r} matches {hits}")
    return hits[0]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", required=True)
    ap.add_argument("--dtype", required=True)
    ap.add_argument("--fetch", required=True, help="output directory of the FETCH_SIZE run")
    ap.add_argument("--write", required=True, help="output directory of the WRITE_SIZE run")
    ap.add_argument("--sq", default="", help="output directory of the SQ_* + GRBM_GUI_ACTIVE run")
    ap.add_argument("--l2", default="", help="output directory of the TCC_HIT_sum TCC_MISS_sum run")
    ap.add_argument("--gemm-kernel", default=ROLE_KERNEL["gemm"], help="substring of the gather GEMM's kernel name")
    ap.add_argument("--wgrad-kernel", default=ROLE_KERNEL["wgrad"], help="substring of the weight gradient's kernel name ('' = none)")
    ap.add_argument("--copy-kernel", default="neg_kernel", help="substring of the calibration copy's name (bench.py copies with torch.neg)")
    ap.add_argument("--copy-min-kib", type=float, default=100000.0, help="smallest WRITE_SIZE that identifies the copy")
    ap.add_argument("--profile", default="", help="the summary under profiles/ that quotes this entry")
    args = ap.parse_args()
    fetch = per_kernel(args.fetch)
    write = per_kernel(args.write)
    sq = per_kernel(args.sq) if args.sq else {}
    l2 = per_kernel(args.l2) if args.l2 else {}
    copies = [k for k in write if args.copy_kernel in k and write[k].get("WRITE_SIZE", 0.0) >= args.copy_min_kib]
    if len(copies) != 1:
        raise SystemExit(f"calibration copy not identified: {copies}")
    copy = copies[0]
    scale_r = COPY_BYTES / (fetch[copy]["FETCH_SIZE"] * 1024.0)
    scale_w = COPY_BYTES / (write[copy]["WRITE_SIZE"] * 1024.0)
    print(f"copy: FETCH_SIZE {fetch[copy]['FETCH_SIZE']:.0f} KiB, WRITE_SIZE {write[copy]['WRITE_SIZE']:.0f} KiB per launch "
          f"of 1 GiB in + 1 GiB out -> scale x{scale_r:.3f} / x{scale_w:.3f}\n")
    print("| kernel | dispatches | FETCH_SIZE KiB | WRITE_SIZE KiB | fetched GB | written GB | duration us |")
    print("|---|---|---|---|---|---|---|")
    for k in sorted(fetch, key=lambda k: -fetch[k]["_n"] * fetch[k]["FETCH_SIZE"]):
        w = write.get(k, {}).get("WRITE_SIZE", 0.0)
        if fetch[k]["FETCH_SIZE"] < 1000 and w < 1000:
            continue
        print(f"| `{k}` | {fetch[k]['_n']} | {fetch[k]['FETCH_SIZE']:.0f} | {w:.0f} | {fetch[k]['FETCH_SIZE'] * 1024 * scale_r / 1e9:.3f} "
              f"| {w * 1024 * scale_w / 1e9:.3f} | {fetch[k]['_us']:.1f} |")

    def derived(needle):
        k = the_kernel(fetch, needle)
        rec = {"kernel": k, "dispatches": fetch[k]["_n"],
               "fetch_bytes": round(fetch[k]["FETCH_SIZE"] * 1024 * scale_r),
               "write_bytes": round(write[k]["WRITE_SIZE"] * 1024 * scale_w)}
        rec["traffic_bytes"] = rec["fetch_bytes"] + rec["write_bytes"]
        rec["avg_us_under_counters"] = round(fetch[k]["_us"], 1)
        if sq:
            s = sq[the_kernel(sq, needle)]
            cycles = s["GRBM_GUI_ACTIVE"] / XCDS
            rec["clock_ghz"] = round(cycles / (s["_us"] * 1000.0), 3)
            rec["mfma_busy_frac"] = round(s["SQ_VALU_MFMA_BUSY_CYCLES"] / (SIMDS * cycles), 4)
            rec["counters"] = {c: round(v) for c, v in s.items() if not c.startswith("_")}
        if l2:
            t = l2[the_kernel(l2, needle)]
            rec["l2_hit"] = round(t["TCC_HIT_sum"] / (t["TCC_HIT_sum"] + t["TCC_MISS_sum"]), 4)
        return rec

    roles = {"gemm": derived(args.gemm_kernel)}
    if args.wgrad_kernel:
        roles["wgrad"] = derived(args.wgrad_kernel)
    if sq:
        print("\n| kernel | clock GHz | MFMA busy | SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES | LDS bank conflict / LDS active | L2 hit |")
        print("|---|---|---|---|---|---|")
        for role, rec in roles.items():
            c = rec["counters"]
            print(f"| `{rec['kernel']}` | {rec['clock_ghz']:.2f} | {rec['mfma_busy_frac'] * 100:.1f} % "
                  f"| {c['SQ_WAIT_INST_ANY'] / c['SQ_WAVE_CYCLES'] * 100:.0f} % "
                  f"| {c['SQ_LDS_BANK_CONFLICT'] / max(c['SQ_LDS_IDX_ACTIVE'], 1) * 100:.0f} % "
                  f"| {rec.get('l2_hit', float('nan')) * 100:.0f} % |")
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        table = {}
    entry = {"fetch_scale": round(scale_r, 4), "write_scale": round(scale_w, 4), "profile": args.profile}
    for role, rec in roles.items():
        rec["sources"] = ROLE_SOURCES[role]
        rec["source_digest"] = source_digest(ROLE_SOURCES[role])
        entry[role] = rec
    table[f"{args.workload}_{args.dtype}"] = entry
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)
        f.write("\n")
    for role, rec in roles.items():
        print(f"\n{args.workload}_{args.dtype} {role}: {rec['kernel']}: {rec['fetch_bytes'] / 1e9:.3f} GB fetched + "
              f"{rec['write_bytes'] / 1e9:.3f} GB written = {rec['traffic_bytes'] / 1e9:.3f} GB per launch")


if __name__ == "__main__":
    main()
