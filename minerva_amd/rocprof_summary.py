"""Condenses the databases rocprofv3 writes (rocpd, SQLite) into the short text tables kept
under profiles/: one row per (kernel, grid), because the GEMM-family kernels run many problem
shapes under one name and only the grid tells them apart.

  python -m minerva_amd.rocprof_summary trace <dir-or-db> [--by-grid SUBSTR] [--min-share 0.0005]
      per-kernel durations of a `rocprofv3 --kernel-trace --stats` run (microseconds)

  python -m minerva_amd.rocprof_summary counters <dir-or-db> [<dir-or-db> ...] [--only SUBSTR[,SUBSTR...]]
                                        [--trace <dir-or-db>] [--show COUNTER,COUNTER,...]
      per-kernel averages of every counter of one or more `rocprofv3 --pmc` runs (one counter set
      per run), plus, where their counters are present, the derived columns
        cycles     = GRBM_GUI_ACTIVE / 8                        (the counter sums the eight XCDs)
        MFMA busy  = SQ_VALU_MFMA_BUSY_CYCLES / (cycles * SIMDs) (one v_mfma_f32_32x32x2_f32 holds
                                                                  the pipe 64 cycles)
        other VALU = (SQ_INSTS_VALU - SQ_VALU_MFMA_BUSY_CYCLES / 64) * 4 / (cycles * SIMDs)
        waves/SIMD = SQ_WAVE_CYCLES * 4 / (cycles * SIMDs)        (the counter ticks every 4 cycles)
        waiting    = SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES            (share of a wavefront's life spent
                                                                  waiting for an instruction to issue)
      and with --trace the average duration of the same (kernel, grid) in a kernel-trace run and the
      shader clock cycles / duration (two separate runs: an estimate, good to a few percent).

Reads only; needs nothing but the Python standard library."""
import argparse
import collections
import glob
import os
import re
import sqlite3
import sys

SIMDS = 256 * 4  # MI355X: 256 CUs x 4 SIMDs


def short(name):
    name = re.sub(r"\(anonymous namespace\)::", "", name)
    name = re.sub(r"MnvGemmTile<(\d+), (\d+), (\d+), \d+, \d+, \d+, (\d+)>", r"T\1x\4x\3", name)
    name = re.sub(r"^void ", "", name)
    return re.sub(r"\(.*$", "", name)


def open_db(path):
    if os.path.isdir(path):
        found = sorted(glob.glob(os.path.join(path, "**", "*.db"), recursive=True))
        if not found:
            raise SystemExit("no .db under %s" % path)
        path = found[0]
    return sqlite3.connect(path)


def _columns(con, table):
    return [r[1] for r in con.execute("pragma table_info(%s)" % table)]


def trace_rows(con, by_grid=""):
    """{(kernel, grid.x, grid.z): [durations in ns]}; the grid is kept only for kernels whose
    name contains `by_grid` (all kernels when it is "*")."""
    cols = _columns(con, "kernels")
    gx = "grid_size_x" if "grid_size_x" in cols else "grid_x"
    gz = "grid_size_z" if "grid_size_z" in cols else "grid_z"
    agg = collections.defaultdict(list)
    for name, dur, x, z in con.execute("select name, duration, %s, %s from kernels" % (gx, gz)):
        k = short(name)
        keep = by_grid == "*" or (by_grid and by_grid in k)
        agg[(k, x if keep else 0, z if keep else 0)].append(dur)
    return agg


def trace_table(agg, min_share=0.0005):
    total = float(sum(sum(v) for v in agg.values())) or 1.0
    lines = ["%-92s %9s %4s %6s %11s %10s %10s %10s %6s" % (
        "kernel", "grid.x", "z", "calls", "total_us", "avg_us", "min_us", "max_us", "%")]
    for (k, x, z), v in sorted(agg.items(), key=lambda kv: -sum(kv[1])):
        if sum(v) / total < min_share:
            continue
        lines.append("%-92s %9d %4d %6d %11.1f %10.2f %10.2f %10.2f %6.2f" % (
            k[:92], x, z, len(v), sum(v) / 1e3, sum(v) / len(v) / 1e3, min(v) / 1e3, max(v) / 1e3,
            100 * sum(v) / total))
    return "\n".join(lines) + "\n"


def counter_rows(cons, only=""):
    """{(kernel, grid.x, grid.z): {counter: average over the dispatches}} over several runs."""
    vals = collections.defaultdict(lambda: collections.defaultdict(list))
    for con in cons:
        q = "select kernel_name, counter_name, value, grid_size_x, grid_size_z from counters_collection"
        for name, ctr, v, x, z in con.execute(q):
            k = short(name)
            if only and not any(o in k for o in only.split(",")):
                continue
            vals[(k, x, z)][ctr].append(v)
    return {key: {c: sum(v) / len(v) for c, v in d.items()} for key, d in vals.items()}


def counter_table(rows, trace=None, min_cycles=20000, show=None):
    """`show`: the raw counters to print beside the derived columns (None: all of them)."""
    counters = sorted({c for d in rows.values() for c in d})
    derived = []
    have = lambda *names: all(n in counters for n in names)
    if have("GRBM_GUI_ACTIVE"):
        derived.append("cycles")
    if have("GRBM_GUI_ACTIVE", "SQ_VALU_MFMA_BUSY_CYCLES"):
        derived.append("MFMA busy")
    if have("GRBM_GUI_ACTIVE", "SQ_VALU_MFMA_BUSY_CYCLES", "SQ_INSTS_VALU"):
        derived.append("other VALU")
    if have("GRBM_GUI_ACTIVE", "SQ_WAVE_CYCLES"):
        derived.append("waves/SIMD")
    if have("SQ_WAVE_CYCLES", "SQ_WAIT_INST_ANY"):
        derived.append("waiting")
    if trace is not None and have("GRBM_GUI_ACTIVE"):
        derived += ["avg_us", "clock GHz"]
    raw = [c for c in counters if c != "GRBM_GUI_ACTIVE" and (show is None or c in show)]
    head = "%-70s %9s %4s" % ("kernel", "grid.x", "z") + "".join(" %12s" % d for d in derived)
    head += "".join(" %26s" % c for c in raw)
    lines = [head]
    for (k, x, z), d in sorted(rows.items()):
        cyc = d.get("GRBM_GUI_ACTIVE", 0.0) / 8.0
        if "GRBM_GUI_ACTIVE" in d and cyc < min_cycles:
            continue
        cells = []
        for name in derived:
            if name == "cycles":
                cells.append("%12.0f" % cyc)
            elif name == "MFMA busy":
                cells.append("%11.1f%%" % (100 * d.get("SQ_VALU_MFMA_BUSY_CYCLES", 0) / (cyc * SIMDS)))
            elif name == "other VALU":
                other = d.get("SQ_INSTS_VALU", 0) - d.get("SQ_VALU_MFMA_BUSY_CYCLES", 0) / 64.0
                cells.append("%11.1f%%" % (100 * other * 4.0 / (cyc * SIMDS)))
            elif name == "waves/SIMD":
                cells.append("%12.2f" % (d.get("SQ_WAVE_CYCLES", 0) * 4.0 / (cyc * SIMDS)))
            elif name == "waiting":
                cells.append("%11.1f%%" % (100 * d.get("SQ_WAIT_INST_ANY", 0) / max(d.get("SQ_WAVE_CYCLES", 0), 1)))
            elif name == "avg_us":
                dur = trace.get((k, x, z))
                cells.append("%12.2f" % (sum(dur) / len(dur) / 1e3) if dur else "%12s" % "-")
            elif name == "clock GHz":
                dur = trace.get((k, x, z))
                cells.append("%12.2f" % (cyc / (sum(dur) / len(dur) / 1e3) / 1e3) if dur else "%12s" % "-")
        line = "%-70s %9d %4d" % (k[:70], x, z) + "".join(" " + c for c in cells)
        line += "".join(" %26.6g" % d[c] if c in d else " %26s" % "-" for c in raw)
        lines.append(line)
    return "\n".join(lines) + "\n"


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    sub = ap.add_subparsers(dest="what", required=True)
    t = sub.add_parser("trace")
    t.add_argument("db")
    t.add_argument("--by-grid", default="gemm", help='kernels split by grid: name substring, or "*"')
    t.add_argument("--min-share", type=float, default=0.0005)
    c = sub.add_parser("counters")
    c.add_argument("db", nargs="+")
    c.add_argument("--only", default="", help="kernel name substring (several, separated by commas: any of them)")
    c.add_argument("--trace", default=None, help="kernel-trace run of the same command, for durations")
    c.add_argument("--show", default=None, help="comma-separated raw counters to print (default: all)")
    args = ap.parse_args(argv)
    if args.what == "trace":
        sys.stdout.write(trace_table(trace_rows(open_db(args.db), args.by_grid), args.min_share))
    else:
        trace = trace_rows(open_db(args.trace), "*") if args.trace else None
        show = None if args.show is None else set(filter(None, args.show.split(",")))
        sys.stdout.write(counter_table(counter_rows([open_db(p) for p in args.db], args.only), trace,
                                       show=show))


if __name__ == "__main__":
    main()
