"""Text summaries of rocprofv3 result databases (ROCm 7.x writes *_results.db).

    python -m xsched_amd.profile_summary kernels  <results.db>      per-kernel time table
    python -m xsched_amd.profile_summary counter  <results.db>      per-kernel counter averages
"""
import sqlite3
import sys


def kernels(db):
    """One row per (kernel, grid size): launches of different sizes are kept apart."""
    cur = sqlite3.connect(db).cursor()
    q = ("select name, grid_x * grid_y * grid_z, count(*), sum(duration), avg(duration), min(duration), "
         "max(duration) from kernels group by name, grid_x, grid_y, grid_z order by sum(duration) desc")
    out = ["%-8s %-12s %-14s %-10s %-10s %-10s %s" %
           ("calls", "grid_threads", "total_us", "avg_us", "min_us", "max_us", "kernel")]
    for name, grid, calls, total, avg, lo, hi in cur.execute(q):
        out.append("%-8d %-12d %-14.1f %-10.3f %-10.3f %-10.3f %s" %
                   (calls, grid, total / 1e3, avg / 1e3, lo / 1e3, hi / 1e3, name))
    return "\n".join(out)


def counter(db):
    cur = sqlite3.connect(db).cursor()
    q = ("select kernel_name, counter_name, grid_size, count(*), avg(value), min(value), max(value), "
         "avg(duration) from counters_collection group by kernel_name, counter_name, grid_size "
         "order by kernel_name")
    out = ["%-12s %-6s %-14s %-14s %-14s %-12s %-10s %s" %
           ("counter", "n", "avg", "min", "max", "avg_dur_ns", "grid", "kernel")]
    for name, ctr, grid, n, avg, lo, hi, dur in cur.execute(q):
        out.append("%-12s %-6d %-14.1f %-14.1f %-14.1f %-12.0f %-10d %s" % (ctr, n, avg, lo, hi, dur, grid, name))
    return "\n".join(out)


if __name__ == "__main__":
    if len(sys.argv) != 3 or sys.argv[1] not in ("kernels", "counter"):
        print(__doc__)
        sys.exit(2)
    print(kernels(sys.argv[2]) if sys.argv[1] == "kernels" else counter(sys.argv[2]))
