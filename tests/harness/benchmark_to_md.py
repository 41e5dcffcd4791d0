#!/usr/bin/env python3
"""Turns the text hip_benchmark prints into Markdown tables.

    tests/harness/hip_benchmark | python tests/harness/benchmark_to_md.py [--kernel-stats x_kernel_stats.csv]

Reads the row format of the reference's harness (tests/includes/test_config.h:210-226, the one
scripts/benchmark_to_md.py:57-76 of the reference parses):

    Problem size: M=512, N=512, K=512
    Precision: bf16
    <name> <time ms> <TFLOPS> <GB/s> PASS|FAIL <max error> <speedup>

and writes one table each for TFLOPS, speedup over the row named reference_* and, beyond what the reference's
converter has, percent of the MI355X dense matrix-core peak for the precision of the block (a FAIL row is
marked).  With --kernel-stats, the per-kernel durations of a `rocprofv3 --kernel-trace --stats` run
(its *_kernel_stats.csv) are appended as a fourth table."""
import argparse
import csv
import re
import sys
from collections import OrderedDict

# dense MFMA peaks of MI355X in TFLOP/s (TOP/s for int8), keyed by the first word of the "Precision:" line
PEAK_TFLOPS = {"bf16": 2500.0, "fp16": 2500.0, "f16": 2500.0, "fp8": 5000.0, "int8": 5000.0, "i8": 5000.0,
               "fp32": 157.3, "f32": 157.3, "fp64": 78.6}

SIZE = re.compile(r"Problem size: M=(\d+), N=(\d+), K=(\d+)")
PRECISION = re.compile(r"Precision:\s*(\S+)")


def parse(lines):
    """-> OrderedDict{(size, precision): OrderedDict{name: row}}, and the row names in first-seen order"""
    blocks, names = OrderedDict(), []
    size, precision, key = None, None, None
    for raw in lines:
        line = raw.strip()
        m = SIZE.search(line)
        if m:
            size, precision, key = "M=%s, N=%s, K=%s" % m.groups(), None, None
            continue
        m = PRECISION.match(line)
        if m and size:
            precision = m.group(1).lower()
            key = (size, precision)
            blocks.setdefault(key, OrderedDict())
            continue
        cols = line.split()
        if key is None or len(cols) != 7 or cols[4] not in ("PASS", "FAIL"):
            continue
        try:
            row = {"ms": float(cols[1]), "tflops": float(cols[2]), "gbs": float(cols[3]), "ok": cols[4] == "PASS",
                   "max_err": float(cols[5]), "speedup": float(cols[6])}
        except ValueError:
            continue
        blocks[key][cols[0]] = row
        if cols[0] not in names:
            names.append(cols[0])
    return blocks, names


def table(blocks, names, title, cell):
    out = ["## " + title, "", "| Problem size | Precision | " + " | ".join(names) + " |",
           "|---|---|" + "---:|" * len(names)]
    for (size, precision), rows in blocks.items():
        cells = [cell(rows[n], precision) if n in rows else "-" for n in names]
        out.append("| %s | %s | %s |" % (size, precision, " | ".join(cells)))
    return "\n".join(out) + "\n"


def _mark(text, row):
    return text if row["ok"] else text + " (FAIL)"


def tflops_cell(row, precision):
    return _mark("%.3f" % row["tflops"], row)


def speedup_cell(row, precision):
    return _mark("%.2fx" % row["speedup"], row)


def peak_cell(row, precision):
    peak = PEAK_TFLOPS.get(precision)
    return "-" if peak is None else _mark("%.2f %%" % (100.0 * row["tflops"] / peak), row)


def kernel_stats_table(path, top=12):
    out = ["## Kernel durations (rocprofv3 --kernel-trace --stats)", "",
           "| Kernel | Calls | Average (us) | Min (us) | Max (us) | % of GPU time |", "|---|---:|---:|---:|---:|---:|"]
    with open(path, newline="") as f:
        for i, r in enumerate(csv.DictReader(f)):
            if i >= top:
                break
            name = r["Name"]
            name = name if len(name) <= 90 else name[:87] + "..."
            out.append("| `%s` | %s | %.2f | %.2f | %.2f | %.2f |" % (
                name, r["Calls"], float(r["AverageNs"]) / 1e3, float(r["MinNs"]) / 1e3, float(r["MaxNs"]) / 1e3,
                float(r["Percentage"])))
    return "\n".join(out) + "\n"


def render(lines, kernel_stats=None):
    blocks, names = parse(lines)
    if not blocks:
        return "No benchmark rows found.\n"
    parts = ["# GEMM benchmark", "",
             table(blocks, names, "TFLOPS", tflops_cell),
             table(blocks, names, "Speedup over the reference row", speedup_cell),
             table(blocks, names, "Percent of the dense matrix-core peak (MI355X)", peak_cell)]
    if kernel_stats:
        parts.append(kernel_stats_table(kernel_stats))
    failed = [(k, n) for k, rows in blocks.items() for n, r in rows.items() if not r["ok"]]
    parts.append("%d rows, %d failed.\n" % (sum(len(r) for r in blocks.values()), len(failed)))
    return "\n".join(parts)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("input", nargs="?", help="harness output (default: stdin)")
    ap.add_argument("--kernel-stats", help="*_kernel_stats.csv of a rocprofv3 --kernel-trace --stats run")
    args = ap.parse_args()
    lines = open(args.input).read().splitlines() if args.input else sys.stdin.read().splitlines()
    sys.stdout.write(render(lines, args.kernel_stats))


if __name__ == "__main__":
    main()
