#!/usr/bin/env python3
"""Benchmark of the deformable-kernel hot path on one MI355X.

A "step" is one forward + backward of a DeformKernel2d layer's operator
(sample_depthwise: forward, grad-input, grad-rotation, grad-filter) over one
batch of synthetic input resident in HBM, issued through the C ABI of
libdk_hip.so on torch's current stream with preallocated outputs.

Default workload: benchmark configuration 2 -- N=64, C=144, 56x56, 3x3 taps, scope 4x4,
stride 1, pad 1, fp32, rotation ~ N(0, 1).

Prints ONE JSON line: the headline metric (achieved HBM GB/s on the
algorithmic bytes of the step), a `roofline` object for the dominant kernel
(timed with events on the launch stream) and a `cpu_baseline` object (the CPU
oracle, OpenMP, on a bounded slice of the same workload).
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "deformable-kernels_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth

WORKLOADS = {
    # name: (N, C, H, W, k, S, stride, pad, dil, groups, rot_std)
    "cfg2": (64, 144, 56, 56, 3, (4, 4), 1, 1, 1, 1, 1.0),
    "cfg1": (2, 32, 28, 28, 3, (4, 4), 1, 1, 1, 1, 0.5),
    # the per-pixel operator on config 3's layer shape, scope 5 x 5 (what GlobalDeformKernel2d's
    # `fused` route issues, with one rotation per image repeated over the pixels)
    "cfg3_local": (128, 256, 28, 28, 3, (5, 5), 1, 1, 1, 1, 0.5),
}
# config 3 (GlobalDeformKernel2d, run with --dtype fp16): N, C, H, W, k, S, stride, pad -- the layer's
# operator sequence: kernels sampled per image (N-d sampler), per-image depthwise convolution, and back
GLOBAL_WORKLOADS = {"cfg3": (128, 256, 28, 28, 3, (5, 5), 1, 1)}
DTYPES = {"fp32": "float32", "bf16": "bfloat16", "fp16": "float16"}

# Other rows of the operator path, timed per entry point with --workload (not the headline metric).
OTHER_WORKLOADS = {
    # deformable variant, benchmark configuration 4: N, C, H, W, k, S, stride, pad, dil, groups, rot_std, off_std
    "cfg4": ("deform", (64, 512, 28, 28, 3, (4, 4), 2, 1, 1, 1, 0.5, 2.0)),
    # the deformable variant on the headline layer's shape (3136 output pixels per plane)
    "deform_56": ("deform", (64, 144, 56, 56, 3, (4, 4), 1, 1, 1, 1, 0.5, 2.0)),
    # the deformable variant on MobileNetV2's first depthwise stage (112 x 112 planes: wider than 64 columns)
    "deform_112": ("deform", (64, 32, 112, 112, 3, (4, 4), 1, 1, 1, 1, 0.5, 2.0)),
    # ... and on 224 x 224 planes, which do not fit LDS at all (the tensors as large as deform_112's)
    "deform_224": ("deform", (16, 32, 224, 224, 3, (4, 4), 1, 1, 1, 1, 0.5, 2.0)),
    # DeformConv2d (scope = kernel, no rotation tensor: rot_std None) on configuration 4's geometry
    "deform_conv_28": ("deform", (64, 512, 28, 28, 3, (3, 3), 2, 1, 1, 1, None, 2.0)),
    # N-d sampler: data shape [C, s...], points, coordinate range
    "nd_cfg3": ("nd", ((256, 5, 5), 1152, (0.0, 4.0))),             # GlobalDeformKernel2d, config 3
    "nd_cfg5": ("nd", ((64, 32, 32, 32), 1 << 20, (-1.0, 32.0))),   # trilinear volume, config 5, full-volume coords
    "nd_cfg5_unit": ("nd", ((64, 32, 32, 32), 1 << 20, (-1.0, 1.0))),  # the same with config 5's own range [-1, 1]^3
}


# HBM traffic per launch comes from two counter runs (rocprofv3 --pmc FETCH_SIZE, then WRITE_SIZE,
# KiB per dispatch) of this script, summarised by `--traffic-from` into profiles/hbm_traffic_<workload>_
# <dtype>.json together with a hash of the kernel sources they were measured on.  Each counter is
# scaled by what it reads for plain elementwise kernels of known size in the same run (the
# calibration multiply below and the 1 GiB streaming passes).
TRAFFIC_RULES = {  # entry point -> regular expressions; a dispatch belongs to the first entry it matches
    # (the pixel-lanes kernel's fourth template argument says whether it runs the transposed geometry)
    "forward": [r"dk::.*local_pixel_lanes_kernel<[^,]*, \d+, \d+, false", r"dk::.*(local|nhwc)_gather\w*_kernel<[^>]*\bfalse\b",
                r"dk::.*local_forward"],
    "grad_input": [r"dk::.*local_pixel_lanes_kernel<[^,]*, \d+, \d+, true", r"dk::.*(local|nhwc)_gather\w*_kernel<[^>]*\btrue\b",
                   r"dk::.*local_grad_input"],
    "grad_rotation": [r"dk::.*(local|nhwc)_grad_rotation"],
    "grad_filter": [r"dk::.*(local|nhwc)_grad_filter", r"dk::.*reduce_partials"],
}


def kernel_source_hash():
    """sha256 over the kernel sources and the C header: the identity the traffic tables are tied to."""
    import glob
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "deformable-kernels_amd", "csrc")
    files = sorted(glob.glob(os.path.join(csrc, "*.hip")) + glob.glob(os.path.join(csrc, "*.h"))
                   + glob.glob(os.path.join(ROOT, "include", "*.h")))
    for f in files:
        h.update(os.path.basename(f).encode() + b"\0")
        with open(f, "rb") as fh:
            h.update(fh.read())
    return h.hexdigest()


def traffic_file(workload, dtype):
    return os.path.join(ROOT, "profiles", "hbm_traffic_%s_%s.json" % (workload, dtype))


def measured_traffic(workload, dtype, kernel):
    """(HBM bytes per launch, stale) from the tracked counter table of this workload: bytes are None
    where no table exists, the entry point was not matched, or the kernel sources have changed since
    the counters were read (stale = True)."""
    try:
        with open(traffic_file(workload, dtype)) as fh:
            table = json.load(fh)
    except (OSError, ValueError):
        return None, False
    if table.get("kernel_source_sha256") != kernel_source_hash():
        return None, True
    e = table.get("entries", {}).get(kernel)
    if not e:
        return None, False
    return int((e["fetch_kib"] * table["fetch_scale"] + e["write_kib"] * table["write_scale"]) * 1024), False


def summarise_traffic(a):
    """--traffic-from FETCH.db WRITE.db: reduce two rocprofv3 counter databases of `bench.py
    --workload W --dtype D` (one run with --pmc FETCH_SIZE, one with --pmc WRITE_SIZE) to the tracked
    table.  Runs on the CPU; needs no GPU."""
    import re
    import sqlite3
    import subprocess
    N, C, H, W = WORKLOADS[a.workload][:4]
    esz = {"fp32": 4, "bf16": 2, "fp16": 2}[a.dtype]
    x_kib = N * C * H * W * esz / 1024.0
    out = {"workload": a.workload, "dtype": a.dtype, "kernel_source_sha256": kernel_source_hash(),
           "unit": "KiB per call of the entry point, as rocprofv3 reports the counter",
           "commands": ["rocprofv3 --pmc %s -d <dir> -o pmc -- python3 bench.py --workload %s --dtype %s --steps 3 "
                        "--warmup 1 --no-cpu-baseline" % (c, a.workload, a.dtype) for c in ("FETCH_SIZE", "WRITE_SIZE")],
           "entries": {}, "kernels": {}}
    try:
        head = subprocess.run(["git", "-C", ROOT, "rev-parse", "HEAD"], capture_output=True, text=True).stdout.strip()
        dirty = subprocess.run(["git", "-C", ROOT, "status", "--porcelain", "--", "deformable-kernels_amd/csrc", "include"],
                               capture_output=True, text=True).stdout.strip()
        out["git_head"] = head + (" + uncommitted changes to the kernel sources" if dirty else "")
    except OSError:
        out["git_head"] = None
    for counter, path, key in (("FETCH_SIZE", a.traffic_from[0], "fetch"), ("WRITE_SIZE", a.traffic_from[1], "write")):
        rows = sqlite3.connect(path).execute(
            "select kernel_name, value from counters_collection where counter_name = ? order by start", (counter,)).fetchall()
        if not rows:
            sys.exit("%s holds no %s values" % (path, counter))
        # calibration: the elementwise multiplies, in launch order: |x| first, then 1 GiB each
        mul = [v for n, v in rows if "MulFunctor" in n]
        known = [x_kib] + [float(1 << 20)] * (len(mul) - 1)
        out[key + "_scale"] = round(sum(known) / sum(mul), 4)
        out[key + "_calibration"] = {"dispatches": len(mul), "known_kib": round(sum(known), 1), "counter_kib": round(sum(mul), 1),
                                     "first_known_kib": x_kib, "first_counter_kib": mul[0]}
        per_name = {}
        for n, v in rows:
            if "dk::" in n:
                per_name.setdefault(n, []).append(v)
        for n, vs in per_name.items():
            short = re.sub(r"\(.*$", "", n.replace("(anonymous namespace)::", "")).replace("void ", "")
            out["kernels"].setdefault(short, {})[key + "_kib"] = round(sum(vs) / len(vs), 1)
            out["kernels"][short]["dispatches"] = len(vs)
    # entry point = its kernels; a kernel launched k times per call counts k times
    calls = {}
    for short, k in out["kernels"].items():
        for entry, rules in TRAFFIC_RULES.items():
            if any(re.search(r, short) for r in rules):
                calls.setdefault(entry, []).append(k)
                break
    for entry, ks in calls.items():
        base = max(k["dispatches"] for k in ks)
        out["entries"][entry] = {
            "fetch_kib": round(sum(k.get("fetch_kib", 0.0) * k["dispatches"] / base for k in ks), 1),
            "write_kib": round(sum(k.get("write_kib", 0.0) * k["dispatches"] / base for k in ks), 1)}
    dest = a.traffic_out or traffic_file(a.workload, a.dtype)
    with open(dest, "w") as fh:
        json.dump(out, fh, indent=1, sort_keys=True)
        fh.write("\n")
    print("wrote", dest)


def traffic_table(a):
    """--traffic-table: the tracked HBM counter tables profiles/hbm_traffic_*.json as one text
    (profiles/local_dk_hbm_counters.txt).  Runs on the CPU; needs no GPU."""
    import glob
    lines = ["HBM traffic counters of the local deformable-kernel operator, MI355X, one GPU: FETCH_SIZE and WRITE_SIZE per call of each",
             "entry point, from the tables profiles/hbm_traffic_<workload>_<dtype>.json (which bench.py reads for roofline.traffic).", "",
             "Commands (from the repository root, on the GPU box; one counter per run, then the summaries, which need no GPU):",
             "  rocprofv3 --pmc FETCH_SIZE -d /tmp/dk_prof/F -o pmc -- python3 bench.py --workload W --dtype D --steps 3 --warmup 1 --no-cpu-baseline --no-network-pass",
             "  rocprofv3 --pmc WRITE_SIZE -d /tmp/dk_prof/W -o pmc -- python3 bench.py --workload W --dtype D --steps 3 --warmup 1 --no-cpu-baseline --no-network-pass",
             "  python3 bench.py --workload W --dtype D --traffic-from /tmp/dk_prof/F/*/pmc_results.db /tmp/dk_prof/W/*/pmc_results.db",
             "  python3 bench.py --traffic-table", "",
             "Calibration: the same runs hold plain elementwise kernels of known size (one pass over |x|, eleven over 1 GiB, each",
             "reading and writing that much).  WRITE_SIZE reads their size (scale 1.0); FETCH_SIZE reads half of it (scale 2.0).", ""]
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "hbm_traffic_*.json"))):
        with open(path) as fh:
            d = json.load(fh)
        N, C, H, W, k, S, stride, pad, dil, groups = WORKLOADS[d["workload"]][:10]
        Ho, Wo = (H + 2 * pad - dil * (k - 1) - 1) // stride + 1, (W + 2 * pad - dil * (k - 1) - 1) // stride + 1
        esz = {"fp32": 4, "bf16": 2, "fp16": 2}[d["dtype"]]
        per, _, _ = algorithmic_bytes(N, C, H, W, Ho, Wo, k, S, groups, esz)
        lines.append("%s, %s (N=%d C=%d %dx%d k=%d scope %dx%d)   [kernel sources: sha256 %s]" % (
            d["workload"], d["dtype"], N, C, H, W, k, S[0], S[1], str(d.get("kernel_source_sha256", ""))[:12]))
        lines.append("  %-14s %12s %10s %12s %10s %10s %14s" % ("entry point", "FETCH KiB", "x%.1f MB" % d["fetch_scale"], "WRITE KiB", "MB", "total MB", "algorithmic MB"))
        for key in ("forward", "grad_input", "grad_rotation", "grad_filter"):
            e = d["entries"].get(key)
            if not e:
                continue
            fm, wm = e["fetch_kib"] * d["fetch_scale"] * 1024 / 1e6, e["write_kib"] * d.get("write_scale", 1.0) * 1024 / 1e6
            lines.append("  %-14s %12.1f %10.1f %12.1f %10.1f %10.1f %14.1f" % (key, e["fetch_kib"], fm, e["write_kib"], wm, fm + wm, per[key] / 1e6))
        lines.append("  kernels: " + "; ".join(d["kernels"]))
        lines.append("")
    lines += ["(MB = 1e6 bytes; algorithmic = every operand touched once.)  The per-pixel operator with a 5 x 5 scope runs its",
              "grad filter as two launches of 16 scope cells each, so it reads its operands twice; forward / grad input of the 16-bit",
              "types write with the default cache policy since the non-temporal 2-byte stores reached memory as partial lines (WRITE_SIZE",
              "47 % above the tensor's size).  Reads are within a few per cent of the compulsory amount everywhere else: the XCD-aware",
              "block order keeps halo rows and rotation planes in one L2, and the matrix-core grad filter deals its tiles round-robin",
              "to the resident workgroups so that neighbours stage neighbouring tiles together."]
    text = "\n".join(lines) + "\n"
    with open(os.path.join(ROOT, "profiles", "local_dk_hbm_counters.txt"), "w") as fh:
        fh.write(text)
    sys.stdout.write(text)


def summarise_profile(a):
    """--profile-from DB: a text summary of a rocprofv3 database (rocpd sqlite, `-d <dir> -o <name>`) of a
    bench.py run: per-kernel durations, per-kernel counter averages when the run was a --pmc run, and for a
    --kernel-trace run of the default workload the timeline of a step -- each dispatch's duration inside
    the step and the idle gap in front of it.  Runs on the CPU; needs no GPU."""
    import re
    import sqlite3
    cur = sqlite3.connect(a.profile_from).cursor()

    def short(n):
        n = n.replace("(anonymous namespace)::", "").replace("void ", "")
        n = re.sub(r"at::native::", "", n)
        return re.sub(r"\(.*$", "", n)[:100]
    lines = []
    rows = cur.execute("select name, start, end from kernels order by start").fetchall()
    if rows:
        stat = {}
        for n, s0, e0 in rows:
            stat.setdefault(short(n), []).append((e0 - s0) / 1e3)
        total = sum(sum(v) for v in stat.values())
        lines.append("%-100s %6s %9s %9s %9s %6s" % ("kernel", "calls", "avg_us", "min_us", "max_us", "pct"))
        for n, v in sorted(stat.items(), key=lambda kv: -sum(kv[1])):
            lines.append("%-100s %6d %9.2f %9.2f %9.2f %6.2f" % (n, len(v), sum(v) / len(v), min(v), max(v), 100 * sum(v) / total))
        # the step's timeline: the longest run of consecutive library dispatches that repeats forward ... grad input
        dk = [(short(n), s0, e0) for n, s0, e0 in rows if "dk::" in n]
        names = [d[0] for d in dk]
        fwd = [i for i, n in enumerate(names) if re.search(TRAFFIC_RULES["forward"][0], n) or re.search(TRAFFIC_RULES["forward"][1], n)]
        period = None
        for i in range(len(fwd) - 1):
            if 2 <= fwd[i + 1] - fwd[i] <= 8:
                period = fwd[i + 1] - fwd[i]
                pattern = names[fwd[i]:fwd[i + 1]]
                break
        has_counters = bool(cur.execute("select count(*) from sqlite_master where name = 'counters_collection'").fetchone()[0]) and \
            bool(cur.execute("select count(*) from counters_collection").fetchone()[0])
        if period and not has_counters:  # (a counter run serialises the dispatches: its gaps say nothing)
            steps = [i for i in fwd if names[i:i + period] == pattern and i + period < len(dk) and names[i + period] == pattern[0]]
            if steps:
                lines.append("")
                lines.append("timeline of a step (%d consecutive steps of the timed loop): duration of each dispatch inside the step, and the" % len(steps))
                lines.append("idle time between the end of the previous dispatch and its start (kernel-trace timestamps)")
                lines.append("%-100s %9s %9s" % ("dispatch", "avg_us", "gap_us"))
                tot_k = tot_g = 0.0
                for j in range(period):
                    dur = sum(dk[i + j][2] - dk[i + j][1] for i in steps) / len(steps) / 1e3
                    gap = sum(dk[i + j][1] - dk[i + j - 1][2] for i in steps if i + j > 0) / len(steps) / 1e3
                    tot_k += dur
                    tot_g += gap
                    lines.append("%-100s %9.2f %9.2f" % (pattern[j], dur, gap))
                span = sum(dk[i + period][1] - dk[i][1] for i in steps) / len(steps) / 1e3
                lines.append("%-100s %9.2f %9.2f   (step to step: %.2f us)" % ("sum", tot_k, tot_g, span))
                lines.append("(Dispatches of one native call follow each other on the device; the gap in front of a call's first")
                lines.append(" dispatch is the host's time between two calls, which the tracer lengthens: without it the host stays")
                lines.append(" ahead of the device and the step takes what bench.py reports.)")
    try:
        crow = cur.execute("select kernel_name, counter_name, count(*), avg(value) from counters_collection "
                           "group by kernel_name, counter_name order by 1, 2").fetchall()
    except sqlite3.Error:
        crow = []
    last = None
    for k, c, n, v in crow:
        if "dk::" not in k:
            continue
        if short(k) != last:
            last = short(k)
            lines.append("")
            lines.append(last)
        lines.append("   %-30s dispatches %-5d average per dispatch %.6g" % (c, n, v))
    text = "\n".join(lines) + "\n"
    if a.profile_out:
        with open(a.profile_out, "a") as fh:
            fh.write(text)
    sys.stdout.write(text)


def algorithmic_bytes(N, C, H, W, Ho, Wo, k, S, groups, esz):
    """Compulsory traffic, every tensor touched once (bytes), per kernel and per step."""
    x = N * C * H * W * esz
    y = N * C * Ho * Wo * esz
    rot = N * groups * k * k * 2 * Ho * Wo * esz
    wt = C * S[0] * S[1] * esz
    per_kernel = {
        "forward": x + rot + wt + y,
        "grad_input": y + rot + wt + x,
        "grad_rotation": y + x + rot + wt + rot,
        "grad_filter": y + x + rot + wt,
        "backward": (y + x + rot + wt) + (x + rot + wt),
    }
    fwd = x + rot + wt + y
    bwd = (y + x + rot + wt) + (x + rot + wt)  # read gout, x, rot, Wt; write gin, grot, gWt
    return per_kernel, fwd, bwd


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", default="cfg2", choices=sorted(WORKLOADS) + sorted(OTHER_WORKLOADS) + sorted(GLOBAL_WORKLOADS) + ["mbv2_dk", "mbv2_net", "layer_cfg2"])
    ap.add_argument("--batch", type=int, default=64, help="batch size of the mbv2_dk workload")
    ap.add_argument("--dtype", default="fp32", choices=sorted(DTYPES))
    ap.add_argument("--shape", default="", help="N,C,H,W,stride: a local-operator layer of that shape (3x3 taps, scope 4x4, "
                    "padding 1) instead of the workload's; for looking at single layers of a network")
    ap.add_argument("--layout", default="nchw", choices=["nchw", "nhwc"],
                    help="memory layout of the tensors of the local-operator workloads (nhwc: the channels-last kernels)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-network-pass", action="store_true",
                    help="skip the MobileNetV2-DK operator pass (the mbv2_dk_* keys of the default run)")
    ap.add_argument("--framework-offset-branch", action="store_true",
                    help="mbv2_net: the layers' offset branch on the framework's convolution (the reference's sequence)")
    ap.add_argument("--kernels", default="", help="comma list restricting the per-kernel timing (tuning aid)")
    ap.add_argument("--traffic-from", nargs=2, metavar=("FETCH_DB", "WRITE_DB"),
                    help="summarise two rocprofv3 counter databases into the tracked traffic table and exit")
    ap.add_argument("--traffic-out", default="", help="where --traffic-from writes (default: profiles/)")
    ap.add_argument("--traffic-table", action="store_true", help="rewrite profiles/local_dk_hbm_counters.txt from the tracked tables")
    ap.add_argument("--profile-from", default="", metavar="DB",
                    help="summarise a rocprofv3 database of a bench.py run (kernel durations, the step's timeline, counters) and exit")
    ap.add_argument("--profile-out", default="", help="append the --profile-from summary to this file as well")
    a = ap.parse_args()
    if a.traffic_from:
        return summarise_traffic(a)
    if a.traffic_table:
        traffic_table(a)
        return
    if a.profile_from:
        return summarise_profile(a)
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU only: every box of this build has one GPU and no "
                 "multi-GPU path exists (the operator shards over the batch with no exchange); "
                 "run with --gpus 1")

    import torch
    from _cases import make_local
    from deformable_kernels.ops.deform_kernel import _lib

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    if a.workload == "mbv2_dk":
        return mobilenet_workload(a)
    if a.workload == "mbv2_net":
        return network_workload(a)
    if a.workload == "layer_cfg2":
        return layer_workload(a)
    if a.workload in OTHER_WORKLOADS:
        return other_workload(a)
    if a.workload in GLOBAL_WORKLOADS:
        return global_workload(a)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    tdtype = getattr(torch, DTYPES[a.dtype])
    N, C, H, W, k, S, stride, pad, dil, groups, rot_std = WORKLOADS[a.workload]
    if a.shape:
        N, C, H, W, stride = [int(v) for v in a.shape.split(",")]
        a.workload = "shape %s" % a.shape
    x, wt, rot, gout, cfg = make_local(N, C, H, W, k, S, stride, pad, dil, groups, rot_std, seed=0, dtype=tdtype)
    Ho, Wo = gout.shape[2], gout.shape[3]
    xg, wg, rg, gg = [t.to(dev) for t in (x, wt, rot, gout)]
    if a.layout == "nhwc":
        xg, rg, gg = [t.contiguous(memory_format=torch.channels_last) for t in (xg, rg, gg)]
    out = torch.empty_like(gg)
    gin = torch.empty_like(xg)
    grot = torch.empty_like(rg)
    gw = torch.empty_like(wg)
    L = _lib.lib()
    desc = _lib.conv_desc(xg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"], groups,
                          layout=_lib.LAYOUT_NHWC if a.layout == "nhwc" else _lib.LAYOUT_NCHW)
    ws, ws_bytes = _lib.workspace(L.dk_sample_depthwise_backward_workspace(desc), dev)
    P = _lib.ptr

    def cur():  # resolved at call time, so launches follow a graph capture's stream
        return _lib.stream_ptr(xg)

    def k_forward():
        _lib.check(L.dk_sample_depthwise_forward(desc, P(xg), P(rg), P(wg), P(out), cur()), "forward")

    def k_grad_input():
        _lib.check(L.dk_sample_depthwise_backward_data(desc, P(gg), P(rg), P(wg), P(gin), cur()), "grad_input")

    def k_grad_rotation():
        _lib.check(L.dk_sample_depthwise_backward_rotation(desc, P(gg), P(xg), P(rg), P(wg), P(grot), P(ws), ws_bytes, cur()),
                   "grad_rotation")

    def k_grad_filter():
        _lib.check(L.dk_sample_depthwise_backward_filter(desc, P(gg), P(xg), P(rg), P(gw), P(ws), ws_bytes, cur()),
                   "grad_filter")

    def k_backward():
        _lib.check(L.dk_sample_depthwise_backward(desc, P(gg), P(xg), P(rg), P(wg), P(gin), P(grot), P(gw),
                                                  P(ws), ws_bytes, cur()), "backward")

    kernels = {"forward": k_forward, "grad_input": k_grad_input, "grad_rotation": k_grad_rotation,
               "grad_filter": k_grad_filter, "backward": k_backward}

    def step():
        if a.kernels:  # tuning aid: time only the named entry points
            for name in a.kernels.split(","):
                kernels[name]()
            return
        k_forward()
        k_backward()  # grad input + grad rotation + grad filter, one native call

    # A plain streaming kernel of known size (|x| read, |x| written): the calibration kernel for
    # the FETCH_SIZE / WRITE_SIZE counters when this script runs under rocprofv3 --pmc.  (An
    # elementwise multiply rather than copy_(), which the runtime turns into its own blit.)
    calib = torch.empty_like(xg)
    torch.mul(xg, 1.0, out=calib)
    del calib
    # Wake-up, untimed and before the warm-up steps: a GPU that has sat idle through the CPU-side
    # input generation runs its first steps below its steady clocks (20 timed steps straight after 5
    # warm-up steps read 13 % low), so the step itself is run in windows of 10 until two consecutive
    # windows agree within 2 % (or 1 s has passed); `wake_ms` says how long that took.
    t_wake = time.perf_counter()
    prev = None
    while time.perf_counter() - t_wake < 1.0:
        t_win = time.perf_counter()
        for _ in range(10):
            step()
        torch.cuda.synchronize()
        win = time.perf_counter() - t_win
        if prev is not None and abs(win - prev) <= 0.02 * prev:
            break
        prev = win
    wake_ms = (time.perf_counter() - t_wake) * 1e3
    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / a.steps

    # per-entry-point launch duration: events on the stream the kernels are launched on
    per_kernel_us = {}
    reps = max(a.steps, 20)
    only = [k for k in a.kernels.split(",") if k]
    for name, fn in kernels.items():
        if only and name not in only:
            continue
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        fn()
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        e1.synchronize()
        per_kernel_us[name] = e0.elapsed_time(e1) * 1e3 / reps

    # measured streaming bandwidth of this GPU: an elementwise pass over 2 x 1 GiB (far beyond the
    # 256 MB memory-side cache)
    big_a = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)
    big_b = torch.empty_like(big_a)
    copy_us = _time_us(lambda: torch.mul(big_a, 1.0, out=big_b), 10)
    copy_gbps = 2 * big_a.numel() * 4 / copy_us / 1e3
    del big_a, big_b


    esz = xg.element_size()
    per_kernel_bytes, fwd_b, bwd_b = algorithmic_bytes(N, C, H, W, Ho, Wo, k, S, groups, esz)
    step_bytes = fwd_b + bwd_b
    gbps = step_bytes / (ms_per_step * 1e-3) / 1e9
    # the dominant kernel: the slowest single launch ("backward" is three of them in one call)
    dominant = max((n for n in per_kernel_us if n != "backward"), key=per_kernel_us.get, default="backward")
    achieved = per_kernel_bytes[dominant] / (per_kernel_us[dominant] * 1e-6) / 1e9

    traffic, traffic_stale = measured_traffic(a.workload, a.dtype, dominant) if a.layout == "nchw" else (None, False)
    result = {
        "metric": "DK fwd+bwd achieved HBM GB/s",
        "value": round(gbps, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "wake_ms": round(wake_ms, 1),
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {"fp32": "f32", "bf16": "bf16", "fp16": "f16"}[a.dtype],
        "data": "synthetic",
        "config": {"workload": "%s: DeformKernel2d op fwd+bwd N=%d C=%d %dx%d k=%d scope=%dx%d stride=%d pad=%d %s%s"
                               % (a.workload, N, C, H, W, k, S[0], S[1], stride, pad, a.dtype,
                                  ", channels-last tensors" if a.layout == "nhwc" else ""),
                   "algorithmic_MB_per_step": round(step_bytes / 1e6, 2)},
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "device_copy_GBps": round(copy_gbps, 1),
        "pct_of_device_copy": round(100.0 * gbps / copy_gbps, 2),
        "images_per_s": round(N / (ms_per_step * 1e-3), 1),
        "layers_per_s": round(1.0 / (ms_per_step * 1e-3), 1),
        "kernel_us": {n: round(v, 2) for n, v in per_kernel_us.items()},
        "roofline": {
            "kernel": dominant,
            "bound": "hbm",
            "achieved": round(achieved, 2),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "algorithmic_bytes": per_kernel_bytes[dominant],
            "traffic": traffic,
        },
    }
    if traffic_stale:
        result["roofline"]["traffic_stale"] = True  # kernel sources changed since the counters were read
    # what the arithmetic type means on this path: the tensors and all sums are `dtype`; where a kernel multiplies on
    # the matrix cores, float32 operands go in as pairs of 16-bit numbers (the measured errors are pinned in tests/)
    if a.dtype == "fp32" and a.layout == "nchw":
        result["arithmetic"] = {
            "tensors_and_sums": "f32",
            "forward, grad_input": "weights formed on v_mfma_f32_16x16x32_f16 from fp16 (hi, lo) pairs of both operands, "
                                   "three products, f32 sums: 2e-7 of the result's scale; the 9 multiply-adds per output in f32",
            "grad_filter": "v_mfma_f32_16x16x16_bf16 on bfloat16 (hi, lo) pairs of both operands, three products, f32 sums: "
                           "5e-6 of the largest element (f32 matrix instructions: 2.4e-7)",
            "grad_rotation": "f32 vector arithmetic throughout",
        }
    # BASELINE's second metric: images/s of the MobileNetV2-DK operator pass (its 17 depthwise DeformKernel2d
    # layers, forward + backward, batch 64, operator calls only) in the same run and dtype
    if a.workload == "cfg2" and a.layout == "nchw" and not a.kernels and not a.no_network_pass:
        del xg, rg, gg, out, gin, grot, ws
        torch.cuda.empty_cache()
        _, net_us, net_bytes = mobilenet_layers(64, a.dtype, 10)
        result["mbv2_dk_ms"] = round(net_us / 1e3, 3)
        result["mbv2_dk_images_per_s"] = round(64 / (net_us * 1e-6), 1)
        result["mbv2_dk_GBps"] = round(net_bytes / net_us / 1e3, 1)

    if not a.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(N, C, H, W, k, S, stride, pad, dil, groups, rot_std, esz)
    print(json.dumps(result))


def _time_us(fn, reps):
    import torch
    fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) * 1e3 / reps


def global_workload(a):
    """Forward + backward of GlobalDeformKernel2d's operator sequence (config 3) through the C ABI:
    nd_linear_sample of the N * 9 per-image taps from the [C, 5, 5] scope weights, the per-image
    depthwise convolution, its two gradients, and the sampler's two gradients.  The pooled branch
    (mean, fc, clamp) that predicts the coordinates is framework code in the reference and is not
    part of the step; the coordinates are synthetic, uniform over the scope."""
    import torch
    from deformable_kernels.ops.deform_kernel import _lib
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    tdtype = getattr(torch, DTYPES[a.dtype])
    N, C, H, W, k, S, stride, pad = GLOBAL_WORKLOADS[a.workload]
    taps = k * k
    g = torch.Generator().manual_seed(0)
    x = torch.randn(N, C, H, W, generator=g).to(tdtype).to(dev)
    scope = torch.randn(C, S[0], S[1], generator=g).to(tdtype).to(dev)
    coord = (torch.rand(N * taps, 2, generator=g) * (S[0] - 1)).to(tdtype).to(dev)
    L, P = _lib.lib(), _lib.ptr
    cdesc = _lib.ConvDesc(N, C, H, W, k, k, stride, stride, pad, pad, 1, 1, 1, 1, 1, _lib.dtype_tag(x), 0, 0.0, 0.0)
    oh, ow = ctypes.c_int32(0), ctypes.c_int32(0)
    _lib.check(L.dk_conv_out_size(cdesc, ctypes.byref(oh), ctypes.byref(ow)), "shape")
    gout = torch.randn(N, C, oh.value, ow.value, generator=g).to(tdtype).to(dev)
    ndesc = _lib.nd_desc(scope, coord)
    # the sampled kernels stay as the sampler writes them, [N * 9, C]: the convolution takes them
    # through element strides (image, channel, tap row, tap column), its kernel gradient likewise
    sampled = torch.empty(N * taps, C, dtype=tdtype, device=dev)
    w_img, wstr = sampled, (ctypes.c_int64 * 4)(taps * C, 1, k * C, C)
    out, gin = torch.empty_like(gout), torch.empty_like(x)
    g_sampled, g_scope, g_coord = torch.empty_like(sampled), torch.empty_like(scope), torch.empty_like(coord)
    gw_img = g_sampled
    wf, nf = _lib.workspace(L.dk_nd_linear_sample_forward_workspace(ndesc), dev)
    wd, nd_ = _lib.workspace(L.dk_nd_linear_sample_backward_data_workspace(ndesc), dev)
    order, wo, no_ = None, None, 0
    if L.dk_nd_linear_sample_order_bytes(ndesc):
        order = torch.empty(L.dk_nd_linear_sample_order_bytes(ndesc), dtype=torch.uint8, device=dev)
        wo, no_ = _lib.workspace(L.dk_nd_linear_sample_order_workspace(ndesc), dev)
    st = _lib.stream_ptr(x)

    def k_sample():
        if order is not None:
            _lib.check(L.dk_nd_linear_sample_order(ndesc, P(coord), P(order), P(wo), no_, st), "order")
        _lib.check(L.dk_nd_linear_sample_forward(ndesc, P(scope), P(coord), P(order), P(sampled), P(wf), nf, st), "sample")

    def k_forward():
        _lib.check(L.dk_image_depthwise_forward(cdesc, P(x), P(w_img), wstr, P(out), st), "conv forward")

    def k_grad_input():
        _lib.check(L.dk_image_depthwise_backward_data(cdesc, P(gout), P(w_img), wstr, P(gin), st), "conv grad input")

    def k_grad_kernels():
        _lib.check(L.dk_image_depthwise_backward_weight(cdesc, P(gout), P(x), P(gw_img), wstr, st), "conv grad kernels")

    def k_sample_backward():
        _lib.check(L.dk_nd_linear_sample_backward_data(ndesc, P(g_sampled), P(coord), P(order), P(g_scope), P(wd), nd_, st),
                   "sample grad data")
        _lib.check(L.dk_nd_linear_sample_backward_coord(ndesc, P(g_sampled), P(scope), P(coord), P(order), P(g_coord),
                                                        P(wf), nf, st), "sample grad coord")

    kernels = {"sample_kernels": k_sample, "forward": k_forward, "grad_input": k_grad_input,
               "grad_kernels": k_grad_kernels, "sample_backward": k_sample_backward}

    def step():
        for fn in kernels.values():
            fn()

    calib = torch.empty_like(x)
    torch.mul(x, 1.0, out=calib)
    del calib
    t_wake, prev = time.perf_counter(), None
    while time.perf_counter() - t_wake < 1.0:
        t_win = time.perf_counter()
        for _ in range(10):
            step()
        torch.cuda.synchronize()
        win = time.perf_counter() - t_win
        if prev is not None and abs(win - prev) <= 0.02 * prev:
            break
        prev = win
    wake_ms = (time.perf_counter() - t_wake) * 1e3
    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(a.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / a.steps
    us = {name: _time_us(fn, max(a.steps, 20)) for name, fn in kernels.items()}
    e = x.element_size()
    bx, by, bw = x.numel() * e, gout.numel() * e, w_img.numel() * e
    small = (sampled.numel() + scope.numel() + coord.numel()) * e
    nbytes = {"sample_kernels": small + 2 * bw, "forward": bx + bw + by, "grad_input": by + bw + bx,
              "grad_kernels": by + bx + bw, "sample_backward": 2 * small + 2 * bw}
    step_bytes = sum(nbytes.values())
    dominant = max(us, key=us.get)
    achieved = nbytes[dominant] / (us[dominant] * 1e-6) / 1e9
    gbps = step_bytes / (ms_per_step * 1e-3) / 1e9
    print(json.dumps({
        "metric": "GlobalDK fwd+bwd achieved HBM GB/s", "value": round(gbps, 2), "unit": "GB/s", "n_gpus": 1,
        "steps": a.steps, "warmup": a.warmup, "wake_ms": round(wake_ms, 1), "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"fp32": "f32", "bf16": "bf16", "fp16": "f16"}[a.dtype], "data": "synthetic",
        "config": {"workload": "%s: GlobalDeformKernel2d operator sequence fwd+bwd N=%d C=%d %dx%d k=%d scope=%dx%d "
                               "stride=%d pad=%d %s" % (a.workload, N, C, H, W, k, S[0], S[1], stride, pad, a.dtype),
                   "algorithmic_MB_per_step": round(step_bytes / 1e6, 2)},
        "pct_of_hbm_peak": round(100.0 * gbps / HBM_PEAK_GBPS, 2),
        "images_per_s": round(N / (ms_per_step * 1e-3), 1),
        "kernel_us": {n: round(v, 2) for n, v in us.items()},
        "roofline": {"kernel": dominant, "bound": "hbm", "achieved": round(achieved, 2), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "algorithmic_bytes": nbytes[dominant],
                     "traffic": None},
    }))


def other_workload(a):
    """Per-entry-point timing of the deformable variant or the N-d sampler (one JSON line,
    `metric` says which; these are not the headline)."""
    import torch
    from _cases import make_deform
    from deformable_kernels.ops.deform_kernel import _lib
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    tdtype = getattr(torch, DTYPES[a.dtype])
    kind, spec = OTHER_WORKLOADS[a.workload]
    L, P = _lib.lib(), _lib.ptr
    reps = max(a.steps, 10)
    us, nbytes = {}, {}
    if kind == "deform":
        N, C, H, W, k, S, stride, pad, dil, groups, rot_std, off_std = spec
        x, wt, rot, off, gout, cfg = make_deform(N, C, H, W, k, S, stride, pad, dil, groups, rot_std or 0.0, off_std,
                                                 seed=0, dtype=tdtype)
        xg, wg, rg, og, gg = [t.to(dev) for t in (x, wt, rot, off, gout)]
        out, gin, grot, goff, gw = [torch.empty_like(t) for t in (gg, xg, rg, og, wg)]
        if rot_std is None:
            rg = None  # NULL at the C ABI: no kernel-space offsets, no rotation tensor read
        desc = _lib.conv_desc(xg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"], groups)
        ws1, n1 = _lib.workspace(L.dk_deformable_sample_depthwise_backward_data_workspace(desc), dev)
        ws2, n2 = _lib.workspace(L.dk_deformable_sample_depthwise_backward_filter_workspace(desc), dev)
        ws3, n3 = _lib.workspace(L.dk_deformable_sample_depthwise_backward_offset_workspace(desc), dev)
        ws4, n4 = _lib.workspace(L.dk_deformable_sample_depthwise_backward_rotation_workspace(desc), dev)
        st = _lib.stream_ptr(xg)
        e = xg.element_size()
        bx, by, br, bo, bw = [(t.numel() * e if t is not None else 0) for t in (xg, gg, rg, og, wg)]
        calls = {
            "forward": (lambda: _lib.check(L.dk_deformable_sample_depthwise_forward(
                desc, P(xg), P(og), P(rg), P(wg), P(out), st), "fwd"), bx + bo + br + bw + by),
            "grad_input": (lambda: _lib.check(L.dk_deformable_sample_depthwise_backward_data(
                desc, P(gg), P(og), P(rg), P(wg), P(gin), P(ws1), n1, st), "gin"), by + bo + br + bw + bx),
            "grad_offset": (lambda: _lib.check(L.dk_deformable_sample_depthwise_backward_offset(
                desc, P(gg), P(xg), P(og), P(rg), P(wg), P(goff), P(ws3), n3, st), "goff"), by + bx + bo + br + bw + bo),
            "grad_rotation": (lambda: _lib.check(L.dk_deformable_sample_depthwise_backward_rotation(
                desc, P(gg), P(xg), P(og), P(rg), P(wg), P(grot), P(ws4), n4, st), "grot"), by + bx + bo + br + bw + br),
            "grad_filter": (lambda: _lib.check(L.dk_deformable_sample_depthwise_backward_filter(
                desc, P(gg), P(xg), P(og), P(rg), P(gw), P(ws2), n2, st), "gw"), by + bx + bo + br + bw),
        }
        if rg is None:
            del calls["grad_rotation"]
        else:
            ws5, n5 = _lib.workspace(L.dk_deformable_sample_depthwise_backward_offset_rotation_workspace(desc), dev)
            calls["grad_offset+rotation, one call"] = (
                lambda: _lib.check(L.dk_deformable_sample_depthwise_backward_offset_rotation(
                    desc, P(gg), P(xg), P(og), P(rg), P(wg), P(goff), P(grot), P(ws5), n5, st), "gcoords"),
                by + bx + 2 * bo + 2 * br + bw)
        label = "%s: deform_sample_depthwise N=%d C=%d %dx%d->%dx%d k=%d scope=%dx%d stride=%d %s%s" % (
            a.workload, N, C, H, W, gg.shape[2], gg.shape[3], k, S[0], S[1], stride, a.dtype,
            "" if rg is not None else ", no rotation tensor")
    else:
        shape, B, (lo, hi) = spec
        g = torch.Generator().manual_seed(0)
        data = torch.randn(*shape, generator=g).to(tdtype).to(dev)
        coord = (torch.rand(B, len(shape) - 1, generator=g) * (hi - lo) + lo).to(tdtype).to(dev)
        go = torch.randn(B, shape[0], generator=g).to(tdtype).to(dev)
        out, gd, gc = torch.empty_like(go), torch.empty_like(data), torch.empty_like(coord)
        desc = _lib.nd_desc(data, coord)
        ws, nb = _lib.workspace(L.dk_nd_linear_sample_backward_data_workspace(desc), dev)
        wf, nf = _lib.workspace(L.dk_nd_linear_sample_forward_workspace(desc), dev)
        st = _lib.stream_ptr(data)
        e = data.element_size()
        bd, bc, bo = data.numel() * e, coord.numel() * e, go.numel() * e
        # each entry point alone (order = NULL: it sorts the points itself when it works on sorted
        # points), then the autograd Function's sequence: order once, the three calls with it
        order, wo, no_ = None, None, 0
        if L.dk_nd_linear_sample_order_bytes(desc):
            order = torch.empty(L.dk_nd_linear_sample_order_bytes(desc), dtype=torch.uint8, device=dev)
            wo, no_ = _lib.workspace(L.dk_nd_linear_sample_order_workspace(desc), dev)

        def whole_step():
            if order is not None:
                _lib.check(L.dk_nd_linear_sample_order(desc, P(coord), P(order), P(wo), no_, st), "order")
            _lib.check(L.dk_nd_linear_sample_forward(desc, P(data), P(coord), P(order), P(out), P(wf), nf, st), "fwd")
            _lib.check(L.dk_nd_linear_sample_backward_data(desc, P(go), P(coord), P(order), P(gd), P(ws), nb, st), "gd")
            _lib.check(L.dk_nd_linear_sample_backward_coord(desc, P(go), P(data), P(coord), P(order), P(gc), P(wf), nf, st),
                       "gc")

        calls = {
            "forward": (lambda: _lib.check(L.dk_nd_linear_sample_forward(
                desc, P(data), P(coord), P(None), P(out), P(wf), nf, st), "fwd"), bd + bc + bo),
            "grad_data": (lambda: _lib.check(L.dk_nd_linear_sample_backward_data(
                desc, P(go), P(coord), P(None), P(gd), P(ws), nb, st), "gd"), bo + bc + bd),
            "grad_coord": (lambda: _lib.check(L.dk_nd_linear_sample_backward_coord(
                desc, P(go), P(data), P(coord), P(None), P(gc), P(wf), nf, st), "gc"), bo + bd + bc + bc),
            "forward+backward, one sort": (whole_step, 2 * (bd + bc + bo) + bo + bd + 2 * bc),
        }
        label = "%s: nd_linear_sample data=%s points=%d %s" % (a.workload, list(shape), B, a.dtype)
    for name, (fn, nb_) in calls.items():
        us[name] = _time_us(fn, reps)
        nbytes[name] = nb_
    total_us = sum(v for k_, v in us.items() if "+" not in k_)
    extra = {}
    if "grad_offset+rotation, one call" in us:  # the Function's backward: both coordinate gradients from one call
        extra["sum_with_one_call_us"] = round(total_us - us["grad_offset"] - us["grad_rotation"]
                                              + us["grad_offset+rotation, one call"], 2)
    print(json.dumps({
        "metric": "per-entry-point time (secondary workload, not the headline)",
        "config": {"workload": label},
        "kernel_us": {k_: round(v, 2) for k_, v in us.items()},
        "algorithmic_GBps": {k_: round(nbytes[k_] / (us[k_] * 1e-6) / 1e9, 1) for k_ in us},
        "sum_us": round(total_us, 2), **extra,
        "n_gpus": 1, "dtype": a.dtype, "data": "synthetic",
    }))


# The 17 depthwise 3x3 layers of MobileNetV2 at 224 x 224 (channels, input size, stride), each
# replaced by DeformKernel2d with a 4 x 4 scope (benchmark configuration 5, operator calls only).
MBV2_DW_LAYERS = [(32, 112, 1), (96, 112, 2), (144, 56, 1), (144, 56, 2), (192, 28, 1), (192, 28, 1), (192, 28, 2),
                  (384, 14, 1), (384, 14, 1), (384, 14, 1), (384, 14, 1), (576, 14, 1), (576, 14, 1), (576, 14, 2),
                  (960, 7, 1), (960, 7, 1), (960, 7, 1)]


def layer_workload(a):
    """A whole LocalDeformKernel2d layer of config 2's shape through the modules and autograd:
    the 3x3 offset branch (rotation_conv), the 'scope' clamp and the operator, forward + backward.
    Times the reference's sequence (library convolution, clamp as tensor ops) against the
    library's own offset-branch kernels and the clamp inside the operator."""
    import torch
    from deformable_kernels.modules import LocalDeformKernel2d
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    N, C, H = a.batch, 144, 56
    tdtype = getattr(torch, DTYPES[a.dtype])
    m = LocalDeformKernel2d((4, 4), C, C, 3, 1, 1, 1, C, 1, False, "scope").to(dev)
    torch.nn.init.normal_(m.rotation_conv.weight, std=0.01)
    m = m.to(tdtype)
    x = torch.randn(N, C, H, H, device=dev).to(tdtype).requires_grad_()
    gout = torch.randn(N, C, H, H, device=dev).to(tdtype)

    def timed(fn):
        for _ in range(a.warmup):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(a.steps):
            fn()
        e1.record()
        e1.synchronize()
        return round(e0.elapsed_time(e1) * 1e3 / a.steps, 1)

    def step():
        m(x).backward(gout)

    def forward():
        with torch.no_grad():
            m(x)

    def branch():
        r = m.rotation_conv(x)
        r.backward(torch.ones_like(r))

    res = {}
    for name, native, fused in (("reference_sequence", False, False), ("clamp_in_operator", False, True),
                                ("clamp_in_operator+native_offset_branch", True, True)):
        m.native_offset_conv, m.fused_clip = native, fused
        res[name] = {"step_us": timed(step), "forward_us": timed(forward)}
    res["library_offset_branch_alone"] = {"step_us": timed(branch)}
    print(json.dumps({"metric": "LocalDeformKernel2d layer fwd+bwd through the modules (secondary workload)",
                      "config": {"workload": "layer_cfg2: N=%d C=144 56x56 k=3 scope=4x4 rotation_clip='scope' %s" % (N, a.dtype)},
                      "variants": res, "n_gpus": 1, "dtype": a.dtype, "data": "synthetic"}))


def mobilenet_layers(batch, dtype_name, reps):
    """Forward + backward of the 17 deformable-kernel depthwise layers of MobileNetV2-DK, operator calls
    only, each distinct layer shape timed `reps` times: (per-layer rows, microseconds per batch, algorithmic bytes)."""
    import collections
    import torch
    from _cases import make_local
    from deformable_kernels.ops.deform_kernel import _lib
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    tdtype = getattr(torch, DTYPES[dtype_name])
    L, P = _lib.lib(), _lib.ptr
    per_layer, total_us, total_bytes = [], 0.0, 0
    for (C, H, stride), count in collections.Counter(MBV2_DW_LAYERS).items():
        x, wt, rot, gout, cfg = make_local(batch, C, H, H, 3, (4, 4), stride, 1, 1, 1, 0.5, seed=0, dtype=tdtype)
        xg, wg, rg, gg = [t.to(dev) for t in (x, wt, rot, gout)]
        out, gin, grot, gw = [torch.empty_like(t) for t in (gg, xg, rg, wg)]
        desc = _lib.conv_desc(xg, wg, cfg["kernel_size"], cfg["stride"], cfg["padding"], cfg["dilation"], 1)
        ws, nb = _lib.workspace(L.dk_sample_depthwise_backward_workspace(desc), dev)
        st = _lib.stream_ptr(xg)

        def step():
            _lib.check(L.dk_sample_depthwise_forward(desc, P(xg), P(rg), P(wg), P(out), st), "forward")
            _lib.check(L.dk_sample_depthwise_backward(desc, P(gg), P(xg), P(rg), P(wg), P(gin), P(grot), P(gw),
                                                      P(ws), nb, st), "backward")
        us = _time_us(step, reps)
        e = xg.element_size()
        _, fwd_b, bwd_b = algorithmic_bytes(batch, C, H, H, gg.shape[2], gg.shape[3], 3, (4, 4), 1, e)
        per_layer.append({"C": C, "HW": H, "stride": stride, "count": count, "us": round(us, 1),
                          "GBps": round((fwd_b + bwd_b) / us / 1e3, 1)})
        total_us += us * count
        total_bytes += (fwd_b + bwd_b) * count
        del xg, wg, rg, gg, out, gin, grot, gw, ws
    return per_layer, total_us, total_bytes


def mobilenet_workload(a):
    """The MobileNetV2-DK operator pass as a workload of its own (one JSON line; secondary to the headline)."""
    per_layer, total_us, total_bytes = mobilenet_layers(a.batch, a.dtype, max(a.steps // 10, 10))
    print(json.dumps({
        "metric": "MobileNetV2-DK depthwise layers fwd+bwd, operator calls only (secondary workload)",
        "config": {"workload": "mbv2_dk: 17 DeformKernel2d layers, batch %d, scope 4x4, %s" % (a.batch, a.dtype)},
        "images_per_s": round(a.batch / (total_us * 1e-6), 1),
        "ms_per_batch": round(total_us / 1e3, 3),
        "algorithmic_MB": round(total_bytes / 1e6, 1),
        "value": round(total_bytes / total_us / 1e3, 1), "unit": "GB/s",
        "pct_of_hbm_peak": round(100.0 * total_bytes / total_us / 1e3 / HBM_PEAK_GBPS, 2),
        "layers": per_layer, "n_gpus": 1, "dtype": a.dtype, "data": "synthetic",
    }))


def network_workload(a):
    """The whole MobileNetV2-DK network of tests/_mbv2_dk.py (benchmark configuration 5: every depthwise 3 x 3
    convolution a DeformKernel2d with a 4 x 4 scope): forward, cross-entropy, backward and an SGD step on
    synthetic images.  The 1 x 1 convolutions, batch norms and the classifier are the framework's; the
    deformable-kernel layers (operator and, where the library has kernels for the shape, their offset
    branch) are this library's.  One JSON line; secondary to the headline."""
    import torch
    from _mbv2_dk import MobileNetV2DK
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    tdtype = getattr(torch, DTYPES[a.dtype])
    torch.manual_seed(0)
    net = MobileNetV2DK().to(dev).to(tdtype)
    if a.framework_offset_branch:
        for m in net.modules():
            if hasattr(m, "native_offset_conv"):
                m.native_offset_conv = False
    # random labels, nothing to learn, and an untrained network's gradients are large (3e3 on the first offset
    # branch): a step size that leaves the parameters where they are keeps every step's work the same
    opt = torch.optim.SGD(net.parameters(), lr=1e-7, momentum=0.9)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(a.batch, 3, 224, 224, generator=g).to(dev).to(tdtype)
    labels = torch.randint(0, 1000, (a.batch,), generator=g).to(dev)

    def step():
        opt.zero_grad(set_to_none=True)
        loss = torch.nn.functional.cross_entropy(net(x).float(), labels)
        loss.backward()
        opt.step()
        return loss

    for _ in range(max(a.warmup, 3)):
        loss = step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(a.steps):
        loss = step()
    e1.record()
    e1.synchronize()
    ms = e0.elapsed_time(e1) / a.steps
    if not bool(torch.isfinite(loss)):
        sys.exit("the loss is not finite: %r" % float(loss))
    print(json.dumps({
        "metric": "MobileNetV2-DK training step, images/s (secondary workload: the whole network)",
        "config": {"workload": "mbv2_net: MobileNetV2 with 17 DeformKernel2d layers (scope 4x4), 224x224, batch %d, %s, "
                               "forward + loss + backward + SGD step%s" % (
                                   a.batch, a.dtype, ", offset branch on the framework's convolution" if a.framework_offset_branch else "")},
        "images_per_s": round(a.batch / (ms * 1e-3), 1), "ms_per_step": round(ms, 3), "steps": a.steps,
        "n_gpus": 1, "dtype": a.dtype, "data": "synthetic",
    }))


def cpu_baseline(N, C, H, W, k, S, stride, pad, dil, groups, rot_std, esz):
    """The CPU oracle (a port of the reference's arithmetic; the reference has no CPU path),
    OpenMP over the host cores, fp32, on the first `n` images of the same seeded workload."""
    from _cases import make_local
    from oracle import dk_oracle as orc
    n = min(N, 16)
    x, wt, rot, gout, cfg = make_local(n, C, H, W, k, S, stride, pad, dil, groups, rot_std, seed=0)
    xs, ws_, rs, gs = [t.numpy() for t in (x, wt, rot, gout)]
    # The threads this job may use: the OpenMP default (OMP_NUM_THREADS where the host sets a CPU share
    # for the job) bounded by the CPUs this process may run on; `host_cpus` is the whole machine.
    try:
        allowed = len(os.sched_getaffinity(0))
    except AttributeError:
        allowed = os.cpu_count() or 1
    threads = max(1, min(orc.max_threads(), allowed))
    orc.set_threads(threads)
    model = ""
    try:
        with open("/proc/cpuinfo") as fh:
            model = next((ln.split(":", 1)[1].strip() for ln in fh if ln.startswith("model name")), "")
    except OSError:
        pass
    # passes over the sample until about 12 s of CPU work are done (at least 3 passes)
    times = []
    t_all = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_all < 12 and len(times) < 200):
        t0 = time.perf_counter()
        orc.sample_depthwise_forward(xs, rs, ws_, **cfg)
        orc.sample_depthwise_backward(gs, xs, rs, ws_, **cfg)
        times.append(time.perf_counter() - t0)
    mean = sum(times) / len(times)
    Ho, Wo = gout.shape[2], gout.shape[3]
    _, fwd_b, bwd_b = algorithmic_bytes(n, C, H, W, Ho, Wo, k, S, groups, 4)
    # one thread, one pass over the first 2 images (the same arithmetic, for the per-core figure)
    orc.set_threads(1)
    t0 = time.perf_counter()
    orc.sample_depthwise_forward(xs[:2], rs[:2], ws_, **cfg)
    orc.sample_depthwise_backward(gs[:2], xs[:2], rs[:2], ws_, **cfg)
    t_one = time.perf_counter() - t0
    orc.set_threads(threads)
    return {
        "value": round((fwd_b + bwd_b) / mean / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "host_cpus": os.cpu_count(),
        "cpus_allowed": allowed,
        "cpu_model": model,
        "one_core_value": round((fwd_b + bwd_b) * 2 / n / t_one / 1e9, 4),
        "kind": "port",
        "sample": "first %d of %d images of the same seeded workload, fwd + 3 grads, fp32, mean of %d passes "
                  "(%.1f s of CPU work, %.3f s per pass, %.1f images/s)"
                  % (n, N, len(times), sum(times), mean, n / mean),
    }


if __name__ == "__main__":
    main()
