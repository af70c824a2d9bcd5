"""Condenses rocprofv3 output of a short bench.py run into the figures the bench line and the
profile notes quote: average launch durations of the attention and norm kernels, and their HBM
traffic per launch from the FETCH_SIZE / WRITE_SIZE counters.

    cd /tmp && export TMPDIR=/tmp
    rocprofv3 --kernel-trace --stats --output-format csv -d OUT/kt -o p -- python3 REPO/bench.py --no-cpu --no-sweep --steps 20 --warmup 5
    rocprofv3 --pmc FETCH_SIZE --kernel-trace --output-format csv -d OUT/fetch -o p -- python3 REPO/bench.py --no-cpu --no-sweep --steps 5 --warmup 2
    rocprofv3 --pmc WRITE_SIZE --kernel-trace --output-format csv -d OUT/write -o p -- python3 REPO/bench.py --no-cpu --no-sweep --steps 5 --warmup 2
    python3 REPO/lightning-attention_amd/benchmarks/profile_summary.py --kt OUT/kt --fetch OUT/fetch --write OUT/write \
        --out REPO/profiles/la_step_b4_h32_n8192_d128_bf16.counters.json

Both counters report KiB per dispatch.  They are scaled by what they read for a kernel of known
size in the same run: PyTorch's float32 -> bfloat16 cast of the run's largest tensor (bench.py
makes its inputs that way; [4, 32, 8192, 128] unless --cast-elements says otherwise), which reads
4 and writes 2 bytes per element.  The run must not hold larger casts (so: --no-sweep, or --shape).
"""
import argparse
import collections
import csv
import glob
import json
import os
import re
import statistics

CAST_ELEMENTS = 4 * 32 * 8192 * 128  # the largest tensor bench.py casts in a --no-sweep run


def classify(name):
    """Short key of a kernel this repository launches (or of the calibration cast), None for others."""
    if "bfloat16_copy_kernel" in name:
        return "cast_f32_to_bf16"
    if "la_sweep_pipe_both_kernel" in name:
        return "sweep_both"
    if "la_sweep_pipe_kernel" in name:
        # la_sweep_pipe_kernel<T, DKP, NF, NH, REVERSE, DECAY, DENSE>, mangled or demangled
        m = (re.search(r"Li(\d+)ELi(\d)ELi(\d)ELb(\d)E", name)
             or re.search(r"<[^,]+, *(\d+), *(\d), *(\d), *(true|false|0|1)", name))
        if not m:
            return "sweep_pipe"
        dkp, rev, wide, whole = int(m.group(1)), m.group(4) in ("1", "true"), m.group(3) == "2", m.group(3) == "3"
        key = ("reverse" if rev else "forward") + ("_all" if whole else "_pair" if rev and wide else "_wide" if wide else "")
        return key if dkp <= 128 else "d%d_%s" % (dkp, key)
    if "la_state_scan" in name:
        return "state_scan"
    if "norm_gate_fwd" in name:
        return "norm_gate_fwd"
    if "norm_gate_bwd" in name:
        return "norm_gate_bwd"
    if "norm_gate_reduce" in name:
        return "norm_gate_reduce"
    if "silu" in name.lower():
        return "torch_silu_bwd" if "backward" in name.lower() else "torch_silu"
    if "srms_fwd" in name:
        return "srms_fwd"
    if "srms_bwd" in name:
        return "srms_bwd"
    return None


def counter_means(folder, counter):
    vals = collections.defaultdict(list)
    for path in glob.glob(os.path.join(folder, "**", "*counter_collection.csv"), recursive=True):
        for r in csv.DictReader(open(path)):
            key = classify(r["Kernel_Name"])
            if key and r["Counter_Name"] == counter:
                vals[key].append(float(r["Counter_Value"]))
    # the cast runs on tensors of several sizes: keep the largest ones (the calibration size)
    if vals.get("cast_f32_to_bf16"):
        top = max(vals["cast_f32_to_bf16"])
        vals["cast_f32_to_bf16"] = [v for v in vals["cast_f32_to_bf16"] if v > 0.9 * top]
    return {k: statistics.fmean(v) for k, v in vals.items()}, {k: len(v) for k, v in vals.items()}


def durations(folder):
    vals = collections.defaultdict(list)
    for path in glob.glob(os.path.join(folder, "**", "*kernel_trace.csv"), recursive=True):
        for r in csv.DictReader(open(path)):
            key = classify(r["Kernel_Name"])
            if key:
                vals[key].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    return {k: {"calls": len(v), "avg_us": round(statistics.fmean(v), 1), "min_us": round(min(v), 1),
                "median_us": round(statistics.median(v), 1), "max_us": round(max(v), 1)} for k, v in vals.items()}


def kernel_names(folder):
    """The kernel names behind each key, as the trace spells them."""
    names = collections.defaultdict(set)
    for path in glob.glob(os.path.join(folder, "**", "*kernel_trace.csv"), recursive=True):
        for r in csv.DictReader(open(path)):
            key = classify(r["Kernel_Name"])
            if key:
                names[key].add(r["Kernel_Name"])
    return {k: sorted(v) for k, v in names.items()}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--kt")
    ap.add_argument("--fetch")
    ap.add_argument("--write")
    ap.add_argument("--out", required=True)
    ap.add_argument("--cast-elements", type=int, default=CAST_ELEMENTS)
    ap.add_argument("--git-head", default=None, help="commit the run was made at (the GPU box holds no .git)")
    a = ap.parse_args()
    cast_read, cast_write = 4 * a.cast_elements, 2 * a.cast_elements
    res = collections.defaultdict(dict)
    if a.kt:
        for k, v in durations(a.kt).items():
            res[k]["duration"] = v
    if a.fetch and a.write:
        fetch, nf = counter_means(a.fetch, "FETCH_SIZE")
        write, _ = counter_means(a.write, "WRITE_SIZE")
        fs = cast_read / (fetch["cast_f32_to_bf16"] * 1024.0)
        ws = cast_write / (write["cast_f32_to_bf16"] * 1024.0)
        res["calibration"] = {"kernel": "float32 -> bfloat16 cast of %d elements" % a.cast_elements, "fetch_scale": round(fs, 4),
                              "write_scale": round(ws, 4), "FETCH_SIZE_KiB": round(fetch["cast_f32_to_bf16"], 1),
                              "WRITE_SIZE_KiB": round(write["cast_f32_to_bf16"], 1)}
        for k in fetch:
            if k == "cast_f32_to_bf16" or k not in write:
                continue
            rd, wr = fetch[k] * 1024.0 * fs, write[k] * 1024.0 * ws
            res[k].update({"FETCH_SIZE_KiB": round(fetch[k], 1), "WRITE_SIZE_KiB": round(write[k], 1),
                           "read_bytes": round(rd), "write_bytes": round(wr), "hbm_bytes": round(rd + wr), "dispatches": nf[k]})
    # what the figures are tied to: the kernel sources (bench.py withholds the traffic figures when they change),
    # the commit and the day
    import datetime
    import hashlib
    import subprocess

    here = os.path.dirname(os.path.abspath(__file__))
    root = os.path.dirname(os.path.dirname(here))
    h = hashlib.sha256()
    csrc = os.path.join(os.path.dirname(here), "csrc")
    files = sorted(glob.glob(os.path.join(csrc, "*.hip")) + glob.glob(os.path.join(csrc, "*.h")))
    files.append(os.path.join(root, "include", "lightning_attn_hip.h"))
    for path in files:
        with open(path, "rb") as f:
            h.update(os.path.basename(path).encode() + b"\0" + f.read())
    res["kernel_sources_sha16"] = h.hexdigest()[:16]
    res["git_head"] = a.git_head
    if not res["git_head"]:
        try:
            res["git_head"] = subprocess.run(["git", "-C", root, "rev-parse", "HEAD"], capture_output=True, text=True).stdout.strip() or None
        except OSError:
            res["git_head"] = None
    res["date"] = datetime.date.today().isoformat()
    res["kernels"] = kernel_names(a.kt) if a.kt else {}
    with open(a.out, "w") as f:
        json.dump(res, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps(res, indent=1, sort_keys=True))


if __name__ == "__main__":
    main()
