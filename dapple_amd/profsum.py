"""Per-kernel summary of a rocprofv3 ``--kernel-trace`` rocpd database (``*_results.db``).

    python -m dapple_amd.profsum gpurun_out/prof/bench_results.db
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


if __name__ == "__main__":
    print(summarize(sys.argv[1]))
