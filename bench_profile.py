#!/usr/bin/env python3
"""Profile one workload of bench.py with rocprofv3 and write its summary to profiles/.

    python3 bench_profile.py <workload> [--out-dir prof_out/<workload>]

<workload> is one of bench.py's --workload names (prefill, decode_read, decode_read_int8_gqa8,
wide_routing, pyramid) or `ceilings` (the streaming probes alone).  Three profiler passes run,
each as a process of its own with the program directly after `--`:

    rocprofv3 --kernel-trace --output-format csv -d <dir>/trace -o p -- python3 bench.py --workload <w> --no-cpu-baseline
    rocprofv3 --pmc FETCH_SIZE --output-format csv -d <dir>/fetch -o p -- python3 bench.py --workload <w> --no-cpu-baseline --steps 5 --warmup 2
    rocprofv3 --pmc WRITE_SIZE --output-format csv -d <dir>/write -o p -- python3 bench.py --workload <w> --no-cpu-baseline --steps 5 --warmup 2

Every run also executes the streaming probes of `bench.py` (bench_probe.hip: kernels that read,
write or copy exactly 2 GiB), so each counter is scaled inside its own run by what it reads for a
launch of known traffic.  Rows are keyed by (kernel, grid size): launches of one kernel at
different sizes are never averaged together.  The summary goes to profiles/<workload>.md and ends
in a machine-readable block that bench.py reads for `roofline.traffic`.
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
WORKLOADS = ["prefill", "decode_read", "decode_read_int8_gqa8", "wide_routing", "pyramid", "ceilings"]
PROBE = {"read": "stream_probe_kernel<0, false>", "write": "stream_probe_kernel<1, false>"}


def run_pass(kind: str, out_dir: str, bench_args: list[str]) -> str:
    d = os.path.join(out_dir, kind)
    os.makedirs(d, exist_ok=True)
    flags = {"trace": ["--kernel-trace"], "fetch": ["--pmc", "FETCH_SIZE"], "write": ["--pmc", "WRITE_SIZE"]}[kind]
    cmd = ["rocprofv3", *flags, "--output-format", "csv", "-d", d, "-o", "p", "--",
           "python3", os.path.join(ROOT, "bench.py"), *bench_args]
    env = dict(os.environ, TMPDIR="/tmp")
    with open(os.path.join(d, "log.txt"), "w") as log:
        r = subprocess.run(cmd, cwd="/tmp", env=env, stdout=log, stderr=subprocess.STDOUT, timeout=900)
    if r.returncode != 0:
        raise SystemExit(f"{' '.join(cmd)} failed, see {d}/log.txt")
    return d


def short(name: str) -> str:
    name = name.replace("void ", "").replace("pikv::", "")
    i = name.find("(")
    return name if i < 0 else name[:i]


def read_trace(d: str):
    f = glob.glob(os.path.join(d, "**", "*kernel_trace.csv"), recursive=True)[0]
    rows = collections.defaultdict(list)
    for r in csv.DictReader(open(f)):
        grid = (int(r["Grid_Size_X"]), int(r["Grid_Size_Y"]), int(r["Grid_Size_Z"]))
        rows[(short(r["Kernel_Name"]), grid)].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    return rows


def read_counter(d: str, counter: str):
    f = glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)[0]
    rows = collections.defaultdict(list)
    for r in csv.DictReader(open(f)):
        if r["Counter_Name"] == counter:
            rows[(short(r["Kernel_Name"]), int(r["Grid_Size"]))].append(float(r["Counter_Value"]))
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("workload", choices=WORKLOADS)
    ap.add_argument("--out-dir", default=None)
    args = ap.parse_args()
    w = args.workload
    out_dir = os.path.abspath(args.out_dir or os.path.join(ROOT, "prof_out", w))
    base = ["--calibrate-copy"] if w == "ceilings" else ["--workload", w, "--no-cpu-baseline"]
    short_run = [] if w == "ceilings" else ["--steps", "5", "--warmup", "2"]
    trace = read_trace(run_pass("trace", out_dir, base))
    fetch = read_counter(run_pass("fetch", out_dir, base + short_run), "FETCH_SIZE")
    write = read_counter(run_pass("write", out_dir, base + short_run), "WRITE_SIZE")

    # calibration: the probes move exactly probe_bytes per launch
    probe_bytes = None
    for line in open(os.path.join(out_dir, "trace", "log.txt")):
        if line.startswith("{"):
            j = json.loads(line)
            probe_bytes = (j.get("hbm_ceiling") or {}).get("buffer_bytes") or probe_bytes
            bench_line = j

    probe_threads = probe_bytes // 32768 * 256      # a probe block of 256 threads moves 32 KiB

    def probe_mean(table, key):
        vals = [v for (k, g), vs in table.items() if k == PROBE[key] and g == probe_threads for v in vs]
        return sum(vals) / len(vals) if vals else None
    f_probe, w_probe = probe_mean(fetch, "read"), probe_mean(write, "write")
    f_scale = probe_bytes / (f_probe * 1024) if f_probe else None   # counters are KiB per dispatch
    w_scale = probe_bytes / (w_probe * 1024) if w_probe else None

    lines, machine = [], {}
    total_us = sum(sum(v) for v in trace.values())
    for (name, grid), ts in sorted(trace.items(), key=lambda kv: -sum(kv[1])):
        if not any(s in name for s in ("kernel",)) or name.startswith("at::") or "rocclr" in name:
            continue
        threads = grid[0] * grid[1] * grid[2]
        fv = fetch.get((name, threads))
        wv = write.get((name, threads))
        fb = sum(fv) / len(fv) * 1024 * f_scale if fv and f_scale else None
        wb = sum(wv) / len(wv) * 1024 * w_scale if wv and w_scale else None
        avg = sum(ts) / len(ts)
        tb = (fb or 0) + (wb or 0) if (fb is not None or wb is not None) else None
        lines.append(f"| `{name}` | {grid[0]}x{grid[1]}x{grid[2]} | {len(ts)} | {avg:.1f} | {min(ts):.1f} | {max(ts):.1f} | "
                     f"{'-' if fb is None else f'{fb / 1e6:.1f}'} | {'-' if wb is None else f'{wb / 1e6:.1f}'} | "
                     f"{'-' if tb is None else f'{tb / avg / 1e6:.2f}'} | {100 * sum(ts) / total_us:.1f} |")
        machine[f"{name} @ {threads}"] = {"avg_us": round(avg, 2), "calls": len(ts),
                                          "fetch_bytes": None if fb is None else round(fb),
                                          "write_bytes": None if wb is None else round(wb)}
    md = os.path.join(ROOT, "profiles", f"{w}.md")
    with open(md, "w") as o:
        o.write(f"# rocprofv3 summary: bench.py workload `{w}`\n\n")
        o.write("MI355X (gfx950), ROCm 7.2.0, one GPU.  Made by `python3 bench_profile.py " + w + "`, i.e. three runs from /tmp:\n\n")
        for kind, fl, extra in (("trace", "--kernel-trace", []), ("fetch", "--pmc FETCH_SIZE", short_run), ("write", "--pmc WRITE_SIZE", short_run)):
            o.write(f"    rocprofv3 {fl} --output-format csv -d <dir>/{kind} -o p -- python3 bench.py {' '.join(base + extra)}\n")
        o.write("\nOne row per (kernel, grid size in threads), launches of different sizes are never mixed.  `fetched` / `written` "
                "= FETCH_SIZE / WRITE_SIZE (KiB per dispatch) x 1024 x the factor that makes the same counter, in the same run, read "
                f"{probe_bytes} bytes for one launch of the streaming probe (`stream_probe_kernel<0,false>` reads exactly that, "
                f"`<1,false>` writes it): FETCH_SIZE x {f_scale:.4f}, WRITE_SIZE x {w_scale:.4f}.  TB/s = (fetched + written) / average duration.\n\n")
        o.write("| kernel | grid (threads) | calls | avg us | min us | max us | fetched MB | written MB | TB/s | % of GPU time |\n|---|---|---|---|---|---|---|---|---|---|\n")
        o.write("\n".join(lines) + "\n")
        hc = bench_line.get("hbm_ceiling") if isinstance(bench_line, dict) else None
        if hc:
            o.write("\nStreaming ceilings measured in the kernel-trace run (library access pattern, 2 GiB buffers, GB/s): "
                    + ", ".join(f"{k} {v:.0f}" for k, v in hc.items() if k.endswith("GBps")) + ".\n")
        o.write("\n<!-- machine-readable: " + json.dumps({"workload": w, "fetch_scale": f_scale, "write_scale": w_scale,
                                                         "kernels": machine}) + " -->\n")
    print("wrote", md)


if __name__ == "__main__":
    sys.exit(main())
