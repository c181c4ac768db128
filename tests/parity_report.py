"""Formats the parity report (parity_report.json) that a GPU test run leaves in its output folder:

    python -m tests.parity_report [path] [prefix ...]

prints one markdown table row per recorded check whose name starts with one of the
prefixes (default: the benchmark configurations, "cfg"): the tolerance, the distance of the
GPU result from the fp32 restatement of the reference, its distance from the float64
evaluation, the reference's own distance from float64, and the leg of the gate that passed.
"""
import json
import os
import sys


def rows(report, prefixes):
    for r in report:
        if not any(r["name"].startswith(p) for p in prefixes):
            continue
        fmt = lambda k: f"{r[k]:.2e}" if r.get(k) is not None else "-"
        yield f"| {r['name']} | {r['tol']:.0e} | {fmt('vs_ref')} | {fmt('vs_exact')} | {fmt('ref_vs_exact')} | {r['leg']} |"


def main(argv):
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    path = argv[1] if len(argv) > 1 else os.path.join(root, "gpurun_out", "parity_report.json")
    prefixes = argv[2:] or ["cfg"]
    with open(path) as f:
        report = json.load(f)
    print("| tensor | tolerance | GPU vs fp32 reference | GPU vs float64 | fp32 reference vs float64 | passed by |")
    print("|---|---|---|---|---|---|")
    for line in rows(report, prefixes):
        print(line)


if __name__ == "__main__":
    main(sys.argv)
