"""Per-kernel summary of a rocprofv3 ``--kernel-trace`` rocpd database (``*_results.db``).

    python bench_profsum.py <dir>/bench_results.db
    python bench_profsum.py pmc <dir>/x_counter_collection.csv <kernel name substring>
"""
import re
import sqlite3
import sys


def summarize(path, top=40):
    cur = sqlite3.connect(path).cursor()
    rows = cur.execute("select name, count(*), sum(end-start), avg(end-start), min(end-start), max(end-start) "
                       "from kernels group by name order by 3 desc").fetchall()
    total = sum(r[2] for r in rows)
    out = ["%-100s %7s %12s %10s %10s %10s %6s" % ("kernel", "calls", "total_us", "avg_us", "min_us", "max_us", "pct")]
    for r in rows[:top]:
        name = re.sub(r"\(anonymous namespace\)::", "", r[0])[:100]
        out.append("%-100s %7d %12.1f %10.2f %10.2f %10.2f %6.2f" % (name, r[1], r[2] / 1e3, r[3] / 1e3, r[4] / 1e3,
                                                                    r[5] / 1e3, 100 * r[2] / total))
    out.append("total kernel time us %.1f" % (total / 1e3))
    return "\n".join(out)


def pmc(path, needle):
    """Per-dispatch average of every counter in a rocprofv3 ``--pmc ... --output-format csv`` file, over
    the dispatches whose kernel name contains ``needle`` (counter values are summed over the rows of one
    dispatch: rocprofv3 writes one row per counter instance)."""
    import collections
    import csv
    per = collections.defaultdict(lambda: collections.defaultdict(float))
    names = {}
    with open(path) as f:
        for r in csv.DictReader(f):
            per[r["Dispatch_Id"]][r["Counter_Name"]] += float(r["Counter_Value"])
            names[r["Dispatch_Id"]] = r["Kernel_Name"]
    sel = [d for d in per if needle in names[d]]
    out = ["%d dispatches matching %r" % (len(sel), needle)]
    if sel:
        for c in sorted(per[sel[0]]):
            vals = [per[d][c] for d in sel]
            out.append("%-24s avg %.1f  min %.1f  max %.1f" % (c, sum(vals) / len(vals), min(vals), max(vals)))
            out.append("%-24s per dispatch, in launch order: %s" % ("", " ".join("%.1f" % v for v in vals)))
    return "\n".join(out)


if __name__ == "__main__":
    if sys.argv[1] == "pmc":
        print(pmc(sys.argv[2], sys.argv[3]))
    else:
        print(summarize(sys.argv[1]))
