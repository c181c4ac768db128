"""Text summaries of rocprofv3 runs of bench.py: per-kernel durations, HBM traffic and SQ counters.

    python3 -m lbann_amd.rocprof_summary trace STATS.db [--fetch FETCH.db --write WRITE.db]
                                               [--headline-json OUT.json] [--command "..."]...
    python3 -m lbann_amd.rocprof_summary counters PMC.db [PMC2.db ...] [--match SUBSTR]... [--command "..."]...
    python3 -m lbann_amd.rocprof_summary sequence STATS.db --match SUBSTR [--match SUBSTR]... [--command "..."]...

`trace` prints one markdown table row per (kernel, grid) of a `rocprofv3 --kernel-trace --stats`
database: calls, average and minimum duration, and, for the kernels of the benchmark
configurations, the algorithmic bytes per launch, GB/s and fraction of the 8 TB/s peak.  With the
databases of two counter runs (`--pmc FETCH_SIZE`, `--pmc WRITE_SIZE`) it adds the bytes that
crossed the fabric per launch, each counter scaled by what it reads for the plain 256 MiB copy
kernel that `bench.py --copy-calibration` runs in the same process.  `counters` prints the average
per dispatch of every collected counter for the kernels whose name contains one of the --match
strings.  `sequence` splits the dispatches of the matching kernels by the kernel that ran on the
device immediately before them (what a kernel finds in the caches depends on its predecessor).
All write to stdout; `--command` lines are quoted at the top so that a summary names
the commands that produced it.
"""
import argparse
import json
import re
import sqlite3
import sys

HBM_PEAK_GBS = 8000.0
COPY_KIB = 262144.0  # the calibration copy reads and writes 256 MiB

# kernel-name substring (and, where one kernel serves two workloads, the grid size) ->
# (workload, algorithmic bytes per launch): forward 2 tensors, backward 3, of E elements
_E2, _E3, _E4, _E5A, _E5B = 16777216, 51380224, 33554432, 67108864, 4194304
WORKLOADS = [
    ("sm_fwd_rows<float, 1024, 8, 0", None, "cfg2 softmax fwd 32768x512", 2 * _E2 * 4),
    ("sm_bwd_rows_walk<float, 8, 0", None, "cfg2 softmax bwd (a workgroup walks two rows)", 3 * _E2 * 4),
    ("sm_bwd_rows<float, 1024, 8, 0", None, "cfg2 softmax bwd, one row per workgroup (LBN_NO_BWD_WALK)", 3 * _E2 * 4),
    ("sm_fwd_rows<float, 1024, 8, 1", None, "cfg2 log-softmax fwd", 2 * _E2 * 4),
    ("sm_bwd_rows_walk<float, 8, 1", None, "cfg2 log-softmax bwd", 3 * _E2 * 4),
    # clusters on the 14 x 14 shape (LBN_BN_NO_CHANNEL): 256-thread workgroups, cfg3 takes 512
    ("bn_fwd_cluster<float, 256, 4>", None, "extra: batch norm 128x1024x14x14 fwd, clusters share a channel (LBN_BN_NO_CHANNEL)", 2 * 25690112 * 4),
    ("bn_bwd_cluster<float, 256, 2>", None, "extra: batch norm 128x1024x14x14 bwd, clusters share a channel (LBN_BN_NO_CHANNEL)", 3 * 25690112 * 4),
    ("bn_fwd_cluster_ws<lbn::f16x4, 256, 4>", None, "extra: batch norm fp16 storage 128x1024x14x14 fwd, clusters share a channel (LBN_BN_NO_CHANNEL)", 2 * 25690112 * 2),
    ("bn_bwd_cluster_ws<lbn::f16x4, 256, 4>", None, "extra: batch norm fp16 storage 128x1024x14x14 bwd, clusters share a channel (LBN_BN_NO_CHANNEL)", 3 * 25690112 * 2),
    ("bn_fwd_cluster<float", None, "cfg3 batch norm fwd 64x256x56x56", 2 * _E3 * 4),
    ("bn_bwd_cluster<float", None, "cfg3 batch norm bwd", 3 * _E3 * 4),
    ("bn_fwd_cluster_ws<__half", None, "extra: batch norm fp16 storage fwd 64x256x56x56", 2 * _E3 * 2),
    ("bn_bwd_cluster_ws<__half", None, "extra: batch norm fp16 storage bwd", 3 * _E3 * 2),
    # the other protocol of each storage type, forced with LBN_BN_WAVE_SYNC
    ("bn_fwd_cluster_ws<float", None, "cfg3 batch norm fwd, barrier-free variant (forced)", 2 * _E3 * 4),
    ("bn_bwd_cluster_ws<float", None, "cfg3 batch norm bwd, barrier-free variant (forced)", 3 * _E3 * 4),
    ("bn_fwd_cluster<__half", None, "extra: batch norm fp16 storage fwd, barrier variant (forced)", 2 * _E3 * 2),
    ("bn_bwd_cluster<__half", None, "extra: batch norm fp16 storage bwd, barrier variant (forced)", 3 * _E3 * 2),
    ("ln_fwd_rows<__half", None, "cfg4 layer norm f16 fwd 4096x8192", 2 * _E4 * 2),
    ("ln_bwd_rows<__half", None, "cfg4 layer norm f16 bwd (followed by ln_wgrad_reduce)", 3 * _E4 * 2),
    ("sm_fwd_rows<float, 256, 4, 2", None, "cfg5a channelwise softmax fwd 256x64x4096", 2 * _E5A * 4),
    ("sm_bwd_rows<float, 256, 4, 2", None, "cfg5a channelwise softmax bwd", 3 * _E5A * 4),
    ("sm_fwd_cluster<4, 0, 4, false>", 512, "cfg5b softmax 262144x16 fwd (8 clusters of 64, two rows each)", 2 * _E5B * 4),
    ("sm_bwd_cluster<4, 0, 4, false>", 512, "cfg5b softmax 262144x16 bwd", 3 * _E5B * 4),
    ("sm_fwd_partial", None, "cfg5b softmax 262144x16 fwd, split path, kernel 1 of 2", _E5B * 4),
    ("sm_fwd_apply", None, "cfg5b fwd, split path, kernel 2 of 2", 2 * _E5B * 4),
    ("sm_bwd_partial", None, "cfg5b bwd, split path, kernel 1 of 2", 2 * _E5B * 4),
    ("sm_bwd_apply", None, "cfg5b bwd, split path, kernel 2 of 2", 3 * _E5B * 4),
    ("selftest_copy_pipeline<true>", None, "copy pipeline on cfg3's tensor, batch norm's order of accesses (bench.py --pattern-yardstick)", 2 * _E3 * 4),
    ("selftest_copy_pipeline<false>", None, "copy pipeline on cfg3's tensor, contiguous tiles", 2 * _E3 * 4),
    ("ln_fwd_rows<float, 256, 1>", None, "cfg1 layer norm fwd 1024x128", 2 * 131072 * 4),
    ("ln_bwd_rows<float, 64, 4, 4, false, true>", None, "cfg1 layer norm bwd (weight gradients in the same kernel)", 3 * 131072 * 4),
    ("ln_bwd_rows<float, 64, 4, 4, true", None, "cfg1 layer norm bwd (followed by ln_wgrad_reduce)", 3 * 131072 * 4),
    ("ln_fwd_rows<float, 256, 4>", None, "extra: instance norm fwd 64x256x56x56", 2 * _E3 * 4),
    ("ln_bwd_rows<float, 256, 2, 4, false", None, "extra: instance norm bwd", 3 * _E3 * 4),
    # the same kernels on the storage type whose loads stream (calls beyond the last-level cache)
    ("ln_fwd_rows<lbn::f32s, 256, 4>", None, "extra: instance norm fwd 64x256x56x56 (streaming loads)", 2 * _E3 * 4),
    ("ln_bwd_rows<lbn::f32s, 256, 2, 4, false", None, "extra: instance norm bwd (x through streaming loads)", 3 * _E3 * 4),
    ("sm_fwd_cluster<4, 0, 4, false>", None, "extra: softmax 262144x256 fwd (row clusters)", 2 * 67108864 * 4),
    ("sm_bwd_cluster<4, 0, 4, false>", None, "extra: softmax 262144x256 bwd (row clusters)", 3 * 67108864 * 4),
    ("sm_fwd_cluster<4, 0, 4, true>", None, "extra: softmax 50257x1024 fwd (row clusters, framed 16-byte access)", 2 * 50257 * 1024 * 4),
    ("sm_bwd_cluster<3, 0, 4, true>", None, "extra: softmax 50257x1024 bwd", 3 * 50257 * 1024 * 4),
    ("ln_fwd_stream", None, "extra: instance norm 16x160^3 x 2 fwd (streaming clusters)", 2 * 131072000 * 4),
    ("ln_bwd_stream", None, "extra: instance norm 16x160^3 x 2 bwd", 3 * 131072000 * 4),
    ("ln_fwd_cluster", None, "extra: layer norm over whole samples fwd 802816x64", 2 * _E3 * 4),
    ("ln_bwd_cluster", None, "extra: layer norm over whole samples bwd (followed by ln_wgrad_reduce_wide)", 3 * _E3 * 4),
    ("ebn_fwd_tile", None, "extra: entry-wise batch norm fwd 1048576x64", 2 * 67108864 * 4),
    ("ebn_bwd_tile", None, "extra: entry-wise batch norm bwd", 3 * 67108864 * 4),
    ("sm_fwd_rows_walk<__half, 4, 0", None, "extra: softmax fp16 storage fwd 32768x512 (a workgroup walks two rows)", 2 * _E2 * 2),
    ("sm_bwd_rows_walk_packed<__half, 4, 0", None, "extra: softmax fp16 storage bwd (a workgroup walks two rows)", 3 * _E2 * 2),
    ("sm_fwd_rows<__half, 1024, 4, 0", None, "extra: softmax fp16 storage fwd 32768x512, one row per workgroup (forced)", 2 * _E2 * 2),
    ("sm_bwd_rows<__half, 1024, 4, 0", None, "extra: softmax fp16 storage bwd, one row per workgroup (forced)", 3 * _E2 * 2),
    ("sm_ce_fwd_rows<1024, 8, false>", None, "extra: softmax + cross entropy fwd 32768x512 (x, truth, y)", 3 * _E2 * 4),
    ("sm_ce_bwd_rows<1024, 8, false>", None, "extra: softmax + cross entropy bwd (y, truth, dx)", 3 * _E2 * 4),
    ("ce_fwd_dense", None, "extra: cross entropy fwd 32768x512 (x, truth)", 2 * _E2 * 4),
    ("ce_bwd_dense", None, "extra: cross entropy bwd (x, truth, dx, dtruth)", 4 * _E2 * 4),
    ("esb_fwd_tile", None, "extra: entry-wise scale/bias fwd 1048576x64", 2 * 67108864 * 4),
    ("esb_bwd_tile", None, "extra: entry-wise scale/bias bwd", 3 * 67108864 * 4),
    ("csb_fwd", None, "extra: channel-wise scale/bias fwd 64x256x56x56", 2 * _E3 * 4),
    ("csb_bwd", None, "extra: channel-wise scale/bias bwd", 3 * _E3 * 4),
    ("f64::sm_fwd_rows_f64<0, 1024, 16", None, "extra: softmax fp64 fwd 32768x512", 2 * _E2 * 8),
    ("f64::sm_bwd_rows_parked_f64<0", None, "extra: softmax fp64 bwd (y in registers, dy in registers and LDS)", 3 * _E2 * 8),
    ("f64::rows_stream_f64<1, 0>", None, "extra: softmax fp64 bwd (one workgroup per row, two passes)", 3 * _E2 * 8),
    ("f64::ln_fwd_rows_f64", None, "extra: layer norm fp64 fwd 4096x8192", 2 * _E4 * 8),
    ("f64::ln_bwd_rows_f64", None, "extra: layer norm fp64 bwd (followed by ln_wgrad_reduce_f64)", 3 * _E4 * 8),
    ("f64::bn_fwd_channel_f64", None, "extra: batch norm fp64 64x256x28x28 fwd (one workgroup keeps a channel: x read once)", 2 * 12845056 * 8),
    ("bn_fwd_channel<float, 1024, 8>", None, "extra: batch norm 128x1024x14x14 fwd (one workgroup per channel)", 2 * 25690112 * 4),
    ("bn_bwd_channel<float, 1024, 8>", None, "extra: batch norm 128x1024x14x14 bwd (one workgroup per channel)", 3 * 25690112 * 4),
    ("bn_fwd_channel<lbn::f16x4, 512, 16>", None, "extra: batch norm fp16 storage 128x1024x14x14 fwd (one workgroup per channel)", 2 * 25690112 * 2),
    ("bn_fwd_channel<lbn::f16x4, 1024, 8>", None, "extra: batch norm fp16 storage 128x1024x14x14 fwd (one workgroup per channel)", 2 * 25690112 * 2),
    ("bn_bwd_channel<lbn::f16x4, 1024, 8>", None, "extra: batch norm fp16 storage 128x1024x14x14 bwd (one workgroup per channel)", 3 * 25690112 * 2),
    ("f64::bn_bwd_channel_f64", None, "extra: batch norm fp64 bwd (one workgroup keeps a channel's dy: x read twice, dy once)", 3 * 12845056 * 8),
    ("f64::bn_sums_f64<2, false>", None, "extra: batch norm fp64 64x256x28x28 fwd, kernel 1 of 2 (reads x)", 12845056 * 8),
    ("f64::bn_fwd_apply_f64", None, "extra: batch norm fp64 fwd, kernel 2 of 2 (reads x, writes y)", 2 * 12845056 * 8),
    ("f64::bn_sums_f64<2, true>", None, "extra: batch norm fp64 bwd, kernel 1 of 2 (reads x, dy)", 2 * 12845056 * 8),
    ("f64::bn_bwd_apply_f64", None, "extra: batch norm fp64 bwd, kernel 2 of 2 (reads x, dy, writes dx)", 3 * 12845056 * 8),
    ("grad_sink_quads<true>", None, "extra: gradient buffer, cleared: overwrite 4096x4096", 2 * _E2 * 4),
    ("grad_sink_quads<false>", None, "extra: gradient buffer, ready: accumulate 4096x4096", 3 * _E2 * 4),
]
HEADLINE = "sm_bwd_rows_walk<float, 8, 0"


def _short(name):
    name = re.sub(r"\(.*", "", name).replace("void ", "")
    return name[-100:]


def _rows(db, sql):
    con = sqlite3.connect(db)
    try:
        return con.execute(sql).fetchall()
    finally:
        con.close()


def _workload(name, grid_wgs):
    for sub, wgs, label, nbytes in WORKLOADS:
        if sub in name and (wgs is None or wgs == grid_wgs):
            return label, nbytes
    return None, None


def _counter_by_kernel(db, counter):
    """(kernel name, workgroups) -> average counter value per dispatch."""
    out = {}
    cols = [r[1] for r in _rows(db, "pragma table_info(counters_collection)")]
    gx = "grid_size_x" if "grid_size_x" in cols else ("grid_x" if "grid_x" in cols else None)
    wx = "workgroup_size_x" if "workgroup_size_x" in cols else ("workgroup_x" if "workgroup_x" in cols else None)
    if gx and wx:
        sql = (f"select kernel_name, {gx} / {wx}, avg(value) from counters_collection "
               f"where counter_name='{counter}' group by kernel_name, {gx} / {wx}")
        for n, g, v in _rows(db, sql):
            out[(n, int(g))] = v
    else:
        for n, v in _rows(db, f"select kernel_name, avg(value) from counters_collection "
                              f"where counter_name='{counter}' group by kernel_name"):
            out[(n, None)] = v
    return out


def _lookup(table, name, wgs):
    return table.get((name, wgs), table.get((name, None), 0.0))


def trace(args):
    stats = _rows(args.db, "select name, grid_x / workgroup_x, count(*), avg(end-start), min(end-start) "
                           "from kernels group by name, grid_x / workgroup_x order by sum(end-start) desc")
    fetch = write = None
    ffac = wfac = None
    if args.fetch and args.write:
        fetch, write = _counter_by_kernel(args.fetch, "FETCH_SIZE"), _counter_by_kernel(args.write, "WRITE_SIZE")
        copy_f = [v for (n, _), v in fetch.items() if "MulFunctor" in n]
        copy_w = [v for (n, _), v in write.items() if "MulFunctor" in n]
        if not copy_f or not copy_w:
            sys.exit("the counter runs hold no calibration copy kernel: run bench.py with --copy-calibration")
        ffac, wfac = COPY_KIB / copy_f[0], COPY_KIB / copy_w[0]
    print("# rocprofv3 summary of bench.py\n")
    if args.command:
        print("Commands (from /tmp with TMPDIR=/tmp on the MI355X box; $R is the repository):\n")
        for c in args.command:
            print(f"    {c}")
        print()
    if fetch is not None:
        print(f"Counter scaling from the plain 256 MiB -> 256 MiB copy kernel of the same runs (torch elementwise "
              f"multiply): FETCH_SIZE reads {COPY_KIB / ffac:.0f} KiB for 262144 KiB fetched (factor {ffac:.3f}), "
              f"WRITE_SIZE reads {COPY_KIB / wfac:.0f} KiB for 262144 KiB written (factor {wfac:.3f}). FETCH_SIZE counts "
              f"what the L2s request from the fabric, so reads served by the 256 MB Infinity Cache are included.\n")
    head = "| kernel | workgroups | workload | calls | avg us | min us | algorithmic MB | GB/s (alg/avg) | % of 8 TB/s |"
    sep = "|---|---|---|---|---|---|---|---|---|"
    if fetch is not None:
        head += " fetched MiB | written MiB | traffic / algorithmic |"
        sep += "---|---|---|"
    print(head)
    print(sep)
    headline = None
    for name, wgs, calls, avg, mn in stats:
        wgs = int(wgs)
        label, nbytes = _workload(name, wgs)
        row = f"| `{_short(name)}` | {wgs} | {label or '(helper / torch)'} | {calls} | {avg / 1e3:.2f} | {mn / 1e3:.2f} |"
        if nbytes:
            gbs = nbytes / (avg * 1e-9) / 1e9
            row += f" {nbytes / 1e6:.1f} | {gbs:.0f} | {100 * gbs / HBM_PEAK_GBS:.1f} |"
        else:
            row += " | | |"
        if fetch is not None:
            f = _lookup(fetch, name, wgs) * ffac / 1024
            w = _lookup(write, name, wgs) * wfac / 1024
            row += f" {f:.1f} | {w:.1f} | " + (f"{(f + w) * 1048576 / nbytes:.2f} |" if nbytes else "|")
            if nbytes and HEADLINE in name:
                headline = {"kernel": "sm_bwd_rows_walk<float,8,softmax> at 32768x512",
                            "traffic_bytes_per_launch": (f + w) * 1048576, "fetch_factor": ffac, "write_factor": wfac,
                            "rocprof_avg_us": avg / 1e3}
        elif nbytes and HEADLINE in name:
            headline = {"kernel": "sm_bwd_rows_walk<float,8,softmax> at 32768x512", "rocprof_avg_us": avg / 1e3}
        print(row)
    if args.headline_json and headline:
        with open(args.headline_json, "w") as f:
            json.dump(headline, f, indent=1)


def counters(args):
    print("# rocprofv3 counter summary of bench.py\n")
    if args.command:
        print("Commands (from /tmp with TMPDIR=/tmp on the MI355X box; $R is the repository):\n")
        for c in args.command:
            print(f"    {c}")
        print()
    table = {}
    names = []
    for db in args.db:
        for kernel, counter, calls, value in _rows(
                db, "select kernel_name, counter_name, count(*), avg(value) from counters_collection "
                    "group by kernel_name, counter_name"):
            if args.match and not any(m in kernel for m in args.match):
                continue
            table.setdefault(kernel, {})[counter] = value
            if counter not in names:
                names.append(counter)
    print("Average per dispatch.\n")
    print("| kernel | " + " | ".join(names) + " |")
    print("|---|" + "---|" * len(names))
    for kernel in sorted(table):
        vals = [f"{table[kernel][c]:.4g}" if c in table[kernel] else "" for c in names]
        print(f"| `{_short(kernel)}` | " + " | ".join(vals) + " |")
    # derived ratios where the inputs are there
    print()
    for kernel in sorted(table):
        t = table[kernel]
        notes = []
        if "SQ_WAVE_CYCLES" in t and "SQ_WAIT_ANY" in t and t["SQ_WAVE_CYCLES"]:
            notes.append(f"waves waiting (SQ_WAIT_ANY / SQ_WAVE_CYCLES) {100 * t['SQ_WAIT_ANY'] / t['SQ_WAVE_CYCLES']:.0f} %")
        if "SQ_WAVE_CYCLES" in t and "SQ_WAIT_INST_ANY" in t and t["SQ_WAVE_CYCLES"]:
            notes.append(f"waiting on an instruction (SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES) {100 * t['SQ_WAIT_INST_ANY'] / t['SQ_WAVE_CYCLES']:.0f} %")
        if "SQ_BUSY_CYCLES" in t and "SQ_ACTIVE_INST_VALU" in t and t["SQ_BUSY_CYCLES"]:
            notes.append(f"VALU issue (SQ_ACTIVE_INST_VALU / SQ_BUSY_CYCLES) {t['SQ_ACTIVE_INST_VALU'] / t['SQ_BUSY_CYCLES']:.2f}")
        if notes:
            print(f"* `{_short(kernel)}`: " + "; ".join(notes))


def sequence(args):
    rows = _rows(args.db, "select name, grid_x / workgroup_x, start, end from kernels order by start")
    print("# rocprofv3 kernel trace, dispatches split by the kernel that ran before them\n")
    if args.command:
        print("Commands (from /tmp with TMPDIR=/tmp on the MI355X box; $R is the repository):\n")
        for c in args.command:
            print(f"    {c}")
        print()
    groups = {}
    for i, (name, wgs, start, end) in enumerate(rows):
        if not any(m in name for m in args.match):
            continue
        prev = _short(rows[i - 1][0]) if i else "(first kernel of the process)"
        gap = (start - rows[i - 1][3]) / 1e3 if i else 0.0
        groups.setdefault((_short(name), int(wgs), prev), []).append(((end - start) / 1e3, gap))
    print("| kernel | workgroups | ran after | calls | avg us | median us | min us | max us | median gap to predecessor us |")
    print("|---|---|---|---|---|---|---|---|---|")
    for (name, wgs, prev), v in sorted(groups.items(), key=lambda kv: (kv[0][0], -len(kv[1]))):
        d = sorted(x[0] for x in v)
        g = sorted(x[1] for x in v)
        print(f"| `{name}` | {wgs} | `{prev}` | {len(d)} | {sum(d) / len(d):.2f} | {d[len(d) // 2]:.2f} | {d[0]:.2f} | "
              f"{d[-1]:.2f} | {g[len(g) // 2]:.2f} |")


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="mode", required=True)
    t = sub.add_parser("trace")
    t.add_argument("db")
    t.add_argument("--fetch")
    t.add_argument("--write")
    t.add_argument("--headline-json")
    t.add_argument("--command", action="append", default=[])
    t.set_defaults(fn=trace)
    c = sub.add_parser("counters")
    c.add_argument("db", nargs="+")
    c.add_argument("--match", action="append", default=[])
    c.add_argument("--command", action="append", default=[])
    c.set_defaults(fn=counters)
    q = sub.add_parser("sequence")
    q.add_argument("db")
    q.add_argument("--match", action="append", required=True)
    q.add_argument("--command", action="append", default=[])
    q.set_defaults(fn=sequence)
    args = ap.parse_args()
    args.fn(args)


if __name__ == "__main__":
    main()
