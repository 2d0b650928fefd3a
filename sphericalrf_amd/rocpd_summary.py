"""Text summary of a rocprofv3 result database (the rocpd sqlite file that `rocprofv3 -d DIR -o NAME` leaves as
DIR/NAME_results.db): per kernel the number of dispatches and the mean / min / max duration, and, when the run collected
counters (`--pmc`), the mean of every counter per dispatch.

    python -m sphericalrf_amd.rocpd_summary DIR/NAME_results.db [more.db ...]
"""
import re
import sqlite3
import sys


def _short(name):
    return re.sub(r"\(.*", "", name)[-72:]


def summarise(path, out=sys.stdout):
    con = sqlite3.connect(path)
    rows = con.execute("select name, count(*), avg(end - start), min(end - start), max(end - start), sum(end - start) from kernels "
                       "group by name order by sum(end - start) desc").fetchall()
    total = sum(r[5] for r in rows) or 1
    print("# %s" % path, file=out)
    print("%-74s %6s %11s %11s %11s %6s" % ("kernel", "calls", "avg_us", "min_us", "max_us", "pct"), file=out)
    for name, calls, avg, lo, hi, tot in rows:
        print("%-74s %6d %11.2f %11.2f %11.2f %6.1f" % (_short(name), calls, avg / 1e3, lo / 1e3, hi / 1e3, 100.0 * tot / total), file=out)
    try:
        rows = con.execute("select kernel_name, counter_name, avg(value), count(*) from counters_collection "
                           "group by kernel_name, counter_name order by kernel_name, counter_name").fetchall()
    except sqlite3.Error:
        rows = []
    if rows:
        print(file=out)
        print("%-74s %-22s %18s %6s" % ("kernel", "counter", "mean per dispatch", "n"), file=out)
        for name, counter, mean, n in rows:
            print("%-74s %-22s %18.1f %6d" % (_short(name), counter, mean, n), file=out)
    con.close()


if __name__ == "__main__":
    if len(sys.argv) < 2:
        sys.exit(__doc__)
    for p in sys.argv[1:]:
        summarise(p)
        print()
