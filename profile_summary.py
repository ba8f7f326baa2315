"""Reduces rocprofv3 output (the rocpd SQLite database it writes, `<name>_results.db`) to the text tables kept under
profiles/.

    python profile_summary.py <results.db> [<results.db> ...] [--match substring[,substring...]] [--demangle]

Per database it prints
  * the kernel table: per (kernel, grid) the number of dispatches, the average and the total duration, and the share of
    the run (what `rocprofv3 --kernel-trace --stats` is asked for);
  * when the run collected counters (`--pmc`): per (kernel, grid, counter) the value per dispatch, summed over all
    instances of the counter (XCDs, channels) and averaged over the dispatches.
FETCH_SIZE and WRITE_SIZE are in KiB as the tool reports them; scale them by what the same counter reads for a copy of
known size in the same run (`kernel_bench --filter calibrate`).
"""
import argparse
import sqlite3
import subprocess
import sys


def _suffix(conn, table):
    names = [r[0] for r in conn.execute("select name from sqlite_master where type='table'")]
    found = [n for n in names if n.startswith(table)]
    if not found:
        return None
    return found[0][len(table):]


def _demangle(names):
    try:
        out = subprocess.run(["c++filt"], input="\n".join(n[:-3] if n.endswith(".kd") else n for n in names),
                             stdout=subprocess.PIPE, text=True, check=True).stdout.split("\n")
        return dict(zip(names, out))
    except (OSError, subprocess.CalledProcessError):
        return {n: n for n in names}


def summarize(path, match, demangle, out=sys.stdout, width=110):
    conn = sqlite3.connect(path)
    suf = _suffix(conn, "rocpd_kernel_dispatch")
    if suf is None:
        print("%s: no kernel dispatches recorded" % path, file=out)
        return
    rows = list(conn.execute(
        "select s.kernel_name, d.grid_size_x, d.grid_size_y, d.grid_size_z, count(*), avg(d.end - d.start) / 1000.0, "
        "sum(d.end - d.start) / 1e6 from rocpd_kernel_dispatch%s d join rocpd_info_kernel_symbol%s s on d.kernel_id = s.id "
        "group by s.kernel_name, d.grid_size_x, d.grid_size_y, d.grid_size_z order by 7 desc" % (suf, suf)))
    names = _demangle(sorted({r[0] for r in rows})) if demangle else {r[0]: r[0] for r in rows}
    keep = lambda name: not match or any(m in name or m in names[name] for m in match)
    total = sum(r[6] for r in rows) or 1.0
    print("== %s" % path, file=out)
    print("%-*s %16s %6s %10s %10s %6s" % (width, "kernel", "grid (work-items)", "calls", "avg_us", "total_ms", "share"), file=out)
    for name, gx, gy, gz, calls, avg_us, total_ms in rows:
        if keep(name):
            print("%-*s %16s %6d %10.2f %10.3f %5.1f%%" % (width, names[name][:width], "%dx%dx%d" % (gx, gy, gz), calls, avg_us,
                                                              total_ms, 100 * total_ms / total), file=out)
    psuf = _suffix(conn, "rocpd_pmc_event")
    if psuf is None or conn.execute("select count(*) from rocpd_pmc_event%s" % psuf).fetchone()[0] == 0:
        return
    print("\ncounters: value per dispatch, summed over all instances of the counter, averaged over the dispatches", file=out)
    query = ("select s.kernel_name, d.grid_size_x, d.grid_size_y, d.grid_size_z, p.name, count(distinct d.id), "
             "sum(e.value) / count(distinct d.id) from rocpd_pmc_event%s e join rocpd_info_pmc%s p on e.pmc_id = p.id "
             "join rocpd_kernel_dispatch%s d on e.event_id = d.event_id join rocpd_info_kernel_symbol%s s on d.kernel_id = s.id "
             "group by s.kernel_name, d.grid_size_x, d.grid_size_y, d.grid_size_z, p.name order by 1, 2, 5" % (psuf, psuf, psuf, psuf))
    values = {}
    for name, gx, gy, gz, counter, calls, value in conn.execute(query):
        if keep(name):
            print("%-*s %16s %-28s calls=%5d per_dispatch=%.1f" % (width, names.get(name, name)[:width], "%dx%dx%d" % (gx, gy, gz),
                                                                   counter, calls, value), file=out)
            values.setdefault((name, gx, gy, gz), {})[counter] = value
    derived = [(k, v) for k, v in values.items() if "SQ_VALU_MFMA_BUSY_CYCLES" in v and "SQ_BUSY_CU_CYCLES" in v]
    if derived:
        # a compute unit has four SIMDs, each with its own matrix pipe; SQ_BUSY_CU_CYCLES counts the cycles a unit holds waves
        print("\nmatrix pipe busy = SQ_VALU_MFMA_BUSY_CYCLES / ( 4 * SQ_BUSY_CU_CYCLES )", file=out)
        for (name, gx, gy, gz), v in derived:
            line = "%-*s %16s %5.1f%%" % (width, names.get(name, name)[:width], "%dx%dx%d" % (gx, gy, gz),
                                           100.0 * v["SQ_VALU_MFMA_BUSY_CYCLES"] / (4.0 * v["SQ_BUSY_CU_CYCLES"]))
            if "SQ_WAIT_INST_ANY" in v and "SQ_WAVE_CYCLES" in v:
                line += "   waves waiting on an instruction: %4.1f%% of wave cycles" % (100.0 * v["SQ_WAIT_INST_ANY"] / v["SQ_WAVE_CYCLES"])
            print(line, file=out)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("databases", nargs="+")
    ap.add_argument("--match", default="", help="only kernels whose (demangled) name contains one of these substrings")
    ap.add_argument("--demangle", action="store_true")
    ap.add_argument("--width", type=int, default=110, help="columns kept of a kernel name")
    args = ap.parse_args()
    match = [m for m in args.match.split(",") if m]
    for path in args.databases:
        summarize(path, match, args.demangle, width=args.width)
        print()


if __name__ == "__main__":
    main()
