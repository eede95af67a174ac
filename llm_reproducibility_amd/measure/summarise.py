"""Turns the CSV files of a rocprofv3 run into the short text tables kept under profiles/.

    python -m llm_reproducibility_amd.measure.summarise kernels  DIR [--only tbik::] [--sequence SUBSTRING]
    python -m llm_reproducibility_amd.measure.summarise counters DIR [--kernel SUBSTRING] [--largest N] [--copy-kib KIB] [--by-grid]
    python -m llm_reproducibility_amd.measure.summarise decode   DIR --layers L --steps S

DIR is the directory given to `rocprofv3 -d` (searched recursively for *_kernel_trace.csv / *_counter_collection.csv).

kernels   per kernel: calls, mean / median / min / max duration in microseconds and share of the total, from a
          `--kernel-trace` run.  --sequence NAME also prints that kernel's durations in dispatch order as means of ten
          (what a load phase or a transient after idling looks like).
counters  per kernel and counter: mean over its dispatches, from a `--pmc` run (--largest N: over the N dispatches with
          the largest value only, which leaves out smaller launches of the same kernel).  --copy-kib KIB: the run also
          holds plain device copies of that many KiB (bench.py --calibrate-copy: 49152); FETCH_SIZE and WRITE_SIZE are
          then scaled by what the copy kernel reads for its known size and printed in MB as well.  --by-grid: one entry per
          (kernel, grid size) instead of per kernel, which separates the shapes one kernel was launched on.
decode    a `--kernel-trace` run of `python -m llm_reproducibility_amd.e2e_invariance --layers L ...`: kernel time per
          layer and per step over the last S decode steps, grouped by kind of kernel (the step boundaries are found from
          the q/k-norm + rotary kernel, which runs once per layer and step).
"""
from __future__ import annotations

import argparse
import collections
import csv
import glob
import os
import statistics
import sys


def _find(directory: str, suffix: str):
    hits = sorted(glob.glob(os.path.join(directory, "**", "*" + suffix), recursive=True))
    if not hits:
        raise SystemExit(f"no *{suffix} under {directory}")
    return hits


def _trace(directory: str):
    rows = []
    for path in _find(directory, "_kernel_trace.csv"):
        for r in csv.DictReader(open(path)):
            s, e = int(r["Start_Timestamp"]), int(r["End_Timestamp"])
            rows.append((s, r["Kernel_Name"], (e - s) / 1e3))
    rows.sort()
    return rows


def _short(name: str, width: int = 84) -> str:
    name = name.replace("void ", "")
    return name if len(name) <= width else name[: width - 3] + "..."


def kernels(args) -> int:
    rows = _trace(args.dir)
    by = collections.defaultdict(list)
    for _, k, d in rows:
        if args.only is None or args.only in k:
            by[k].append(d)
    total = sum(sum(v) for v in by.values())
    print("%-84s %7s %10s %10s %10s %10s %8s" % ("kernel", "calls", "mean_us", "median_us", "min_us", "max_us", "share_%"))
    for k, v in sorted(by.items(), key=lambda kv: -sum(kv[1])):
        print("%-84s %7d %10.1f %10.1f %10.1f %10.1f %8.2f" % (_short(k), len(v), statistics.mean(v), statistics.median(v),
                                                           min(v), max(v), 100 * sum(v) / total))
    if args.sequence:
        seq = [d for _, k, d in rows if args.sequence in k]
        if seq:
            big = [d for d in seq if d > 0.6 * max(seq)]
            print(f"\n{args.sequence}: {len(seq)} dispatches, {len(big)} of them above 60 % of the longest; those in dispatch "
                  "order, means of ten (us):")
            print("  " + " ".join("%.0f" % statistics.mean(big[i:i + 10]) for i in range(0, max(len(big) - 9, 1), 10)))
            print("  last 20: mean %.1f us, min %.1f, max %.1f" % (statistics.mean(big[-20:]), min(big[-20:]), max(big[-20:])))
    return 0


def counters(args) -> int:
    agg = collections.defaultdict(lambda: collections.defaultdict(list))
    for path in _find(args.dir, "_counter_collection.csv"):
        for r in csv.DictReader(open(path)):
            key = r["Kernel_Name"] + (f"  [grid {r['Grid_Size']} x wg {r['Workgroup_Size']}]" if args.by_grid else "")
            agg[key][r["Counter_Name"]].append(float(r["Counter_Value"]))
    scale = {}
    if args.copy_kib:
        # the calibration copies are the largest dispatches of the runtime's copy kernel (it also serves small copies)
        for c in ("FETCH_SIZE", "WRITE_SIZE"):
            reads = [max(cs[c]) for k, cs in agg.items() if "copyBuffer" in k and c in cs]
            if reads:
                scale[c] = args.copy_kib / max(reads)
                print(f"plain copy of {args.copy_kib:g} KiB (__amd_rocclr_copyBuffer): {c} reads {max(reads):.0f} -> scale factor {scale[c]:.3f}")
    for k, cs in sorted(agg.items()):
        if args.kernel and args.kernel not in k:
            continue
        print(_short(k, 150))
        for c, vals in sorted(cs.items()):
            vals = sorted(vals)[-args.largest:] if args.largest else vals
            m = statistics.mean(vals)
            extra = ""
            if c in scale:
                extra = f"   x {scale[c]:.3f} KiB = {m * scale[c] * 1024 / 1e6:.1f} MB per dispatch"
            print("  %-30s %14.5g  (%d dispatches)%s" % (c, m, len(vals), extra))
    return 0


_KINDS = [("gemm_single_acc_stream", "batch-invariant mm (streaming kernels; RMSNorm inside where fused)"),
          ("gemm_single_acc", "batch-invariant mm (tile kernels)"),
          ("gemm_tree_strip", "tree GEMM o_proj / down_proj (one-launch kernel; SiLU*up inside where fused)"),
          ("gemm_tree", "tree GEMM o_proj / down_proj (tile kernels)"),
          ("gemm_kernel<", "mm / tree GEMM (small-tile kernel)"),
          ("combine_rmsnorm", "shard combine of the K-cut tree GEMM with the add-RMSNorm of the result"),
          ("combine_", "shard combine of the K-cut tree GEMM"),
          ("attention_decode", "attention (q/k norm + rotary + cache write inside where fused)"),
          ("attention", "attention"), ("rmsnorm", "RMSNorm (+ residual add)"), ("argmax", "token choice (arg-max kernel)"),
          ("silu_mul", "silu_mul"), ("qk_norm_rope", "q/k norm + rotary + cache write")]


def decode(args) -> int:
    rows = _trace(args.dir)
    # a layer pass has exactly one attention launch (prefill or decode)
    att = [i for i, (_, k, _) in enumerate(rows) if "attention" in k]
    need = args.steps * args.layers
    if len(att) < need + 1:
        raise SystemExit(f"only {len(att)} layer passes in the trace, {need} needed")
    # the window starts with the kernels in front of the first attention launch of its first step (embedding lookup, the
    # first norm / projection): everything after the previous step's token choice
    first = att[-need]
    while first > 0 and "argmax" not in rows[first - 1][1]:
        first -= 1
    win = rows[first:]
    per = collections.defaultdict(float)
    launches = collections.Counter()
    for _, k, d in win:
        key = next((lab for sub, lab in _KINDS if sub in k), "library kernels (embedding lookup, position updates, copies)")
        per[key] += d
        launches[key] += 1
    busy = sum(per.values())
    n = args.steps * args.layers
    print(f"kernels {busy / n:6.1f} us per layer ({busy / args.steps:7.1f} us per step), {sum(launches.values()) / n:.1f} launches per layer")
    for key, v in sorted(per.items(), key=lambda kv: -kv[1]):
        print(f"    {key:82s} {v / n:8.1f} us per layer  ({v / args.steps:8.1f} us per step, {launches[key] / args.steps:6.1f} launches)")
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="cmd", required=True)
    k = sub.add_parser("kernels")
    k.add_argument("dir")
    k.add_argument("--only", default=None, help="keep kernels whose name contains this")
    k.add_argument("--sequence", default=None)
    c = sub.add_parser("counters")
    c.add_argument("dir")
    c.add_argument("--kernel", default=None)
    c.add_argument("--largest", type=int, default=0)
    c.add_argument("--copy-kib", type=float, default=0.0)
    c.add_argument("--by-grid", action="store_true")
    d = sub.add_parser("decode")
    d.add_argument("dir")
    d.add_argument("--layers", type=int, required=True)
    d.add_argument("--steps", type=int, required=True)
    args = ap.parse_args(argv)
    return {"kernels": kernels, "counters": counters, "decode": decode}[args.cmd](args)


if __name__ == "__main__":
    sys.exit(main())
