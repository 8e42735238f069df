"""HBM-side traffic per launch of a kernel from two `rocprofv3 --pmc` runs of bench.py, kept in profiles/traffic.json.

The counters FETCH_SIZE and WRITE_SIZE (KiB per dispatch, collected in a run of their own each) are scaled by what
the same counter reads for the plain copy that `bench.py --calibrate-copy` adds (1 GiB read, 1 GiB written per
launch).  Usage, after the two runs

    rocprofv3 --pmc FETCH_SIZE --output-format csv -d /tmp/pmc_fetch -- python3 bench.py --steps 5 --warmup 2 --no-cpu-baseline --calibrate-copy
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d /tmp/pmc_write -- python3 bench.py --steps 5 --warmup 2 --no-cpu-baseline --calibrate-copy

    python -m flexgemm_amd.profile_traffic --workload cfg3 --dtype f16 --kernel gather_gemm_stream_kernel \
        --fetch /tmp/pmc_fetch --write /tmp/pmc_write

writes the entry "cfg3_f16" of profiles/traffic.json (and prints a table of every kernel of the run for the summary
under profiles/).  The entry carries a digest of the kernel's source files; bench.py reports the traffic only while
the digest still matches the sources it runs.
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
# the sources the gather GEMM (forward and dgrad) is built from
GEMM_SOURCES = ["flexgemm_amd/csrc/conv_gemm_stream.hip", "flexgemm_amd/csrc/conv_gemm.hip", "flexgemm_amd/csrc/gemm_device.h",
                "flexgemm_amd/csrc/fgx_common.h", "flexgemm_amd/csrc/tuning.hip"]


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


def per_kernel_mean(directory: str, counter: str):
    """{short kernel name: (dispatches, mean counter value)} over every *_counter_collection.csv below `directory`."""
    acc = {}
    for path in glob.glob(os.path.join(directory, "**", "*counter_collection.csv"), recursive=True):
        with open(path, newline="") as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] != counter:
                    continue
                name = short_name(row["Kernel_Name"])
                cnt, tot = acc.get(name, (0, 0.0))
                acc[name] = (cnt + 1, tot + float(row["Counter_Value"]))
    return {k: (c, t / c) for k, (c, t) in acc.items()}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", required=True)
    ap.add_argument("--dtype", required=True)
    ap.add_argument("--kernel", required=True, help="substring of the dominant kernel's name")
    ap.add_argument("--fetch", required=True, help="output directory of the FETCH_SIZE run")
    ap.add_argument("--write", required=True, help="output directory of the WRITE_SIZE run")
    ap.add_argument("--copy-kernel", default="neg_kernel", help="substring of the calibration copy's name (bench.py copies with torch.neg)")
    ap.add_argument("--copy-min-kib", type=float, default=100000.0, help="smallest WRITE_SIZE that identifies the copy")
    ap.add_argument("--profile", default="", help="the summary under profiles/ that quotes this entry")
    args = ap.parse_args()
    fetch = per_kernel_mean(args.fetch, "FETCH_SIZE")
    write = per_kernel_mean(args.write, "WRITE_SIZE")
    copies = [k for k in write if args.copy_kernel in k and write[k][1] >= args.copy_min_kib]
    if len(copies) != 1:
        raise SystemExit(f"calibration copy not identified: {copies}")
    copy = copies[0]
    scale_r = COPY_BYTES / (fetch[copy][1] * 1024.0)
    scale_w = COPY_BYTES / (write[copy][1] * 1024.0)
    print(f"copy: FETCH_SIZE {fetch[copy][1]:.0f} KiB, WRITE_SIZE {write[copy][1]:.0f} KiB -> scale x{scale_r:.3f} / x{scale_w:.3f}")
    print("| kernel | dispatches | FETCH_SIZE KiB | WRITE_SIZE KiB | fetched GB | written GB |")
    print("|---|---|---|---|---|---|")
    for k in sorted(fetch, key=lambda k: -fetch[k][0] * fetch[k][1]):
        w = write.get(k, (0, 0.0))[1]
        if fetch[k][1] < 1000 and w < 1000:
            continue
        print(f"| `{k}` | {fetch[k][0]} | {fetch[k][1]:.0f} | {w:.0f} | {fetch[k][1] * 1024 * scale_r / 1e9:.3f} | {w * 1024 * scale_w / 1e9:.3f} |")
    mine = [k for k in fetch if args.kernel in k]
    if len(mine) != 1:
        raise SystemExit(f"--kernel matches {mine}")
    k = mine[0]
    fb, wb = fetch[k][1] * 1024 * scale_r, write[k][1] * 1024 * scale_w
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        table = {}
    table[f"{args.workload}_{args.dtype}"] = {
        "kernel": k, "dispatches": fetch[k][0], "fetch_bytes": round(fb), "write_bytes": round(wb),
        "traffic_bytes": round(fb + wb), "fetch_scale": round(scale_r, 4), "write_scale": round(scale_w, 4),
        "sources": GEMM_SOURCES, "source_digest": source_digest(GEMM_SOURCES), "profile": args.profile,
    }
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)
        f.write("\n")
    print(f"{args.workload}_{args.dtype}: {k}: {fb / 1e9:.3f} GB fetched + {wb / 1e9:.3f} GB written = {(fb + wb) / 1e9:.3f} GB per launch")


if __name__ == "__main__":
    main()
