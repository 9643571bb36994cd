"""Summarise a ``rocprofv3`` result database for the int4 kernels.

``rocprofv3 --kernel-trace --stats`` and ``rocprofv3 --pmc ...`` on this ROCm
release write a SQLite database (``*_results.db``).  This prints, per kernel whose
name contains one of the given substrings, the call count and average duration
(kernel trace) or the average counter value per dispatch (PMC run):

    python rocprof_summary.py prof_trace/headline_results.db gemv prepack
"""

from __future__ import annotations

import sqlite3
import sys


def summarise(path: str, needles: list[str]) -> list[str]:
    con = sqlite3.connect(path)
    cur = con.cursor()
    lines = [f"# {path}"]

    def wanted(name: str) -> bool:
        return not needles or any(n in name for n in needles)

    have_pmc = cur.execute("select count(*) from counters_collection").fetchone()[0] > 0
    if have_pmc:
        rows = cur.execute(
            "select kernel_name, counter_name, count(*), avg(value), min(value), max(value) "
            "from counters_collection group by kernel_name, counter_name order by avg(value) desc")
        lines.append("kernel | counter | dispatches | avg | min | max")
        for name, counter, n, avg, lo, hi in rows:
            if wanted(name):
                lines.append(f"{name[:90]} | {counter} | {n} | {avg:.3f} | {lo:.3f} | {hi:.3f}")
    else:
        rows = cur.execute(
            "select name, count(*), avg(end - start), min(end - start), max(end - start), "
            "sum(end - start) from kernels group by name order by sum(end - start) desc")
        lines.append("kernel | calls | avg_us | min_us | max_us | total_us")
        for name, n, avg, lo, hi, tot in rows:
            if wanted(name):
                lines.append(f"{name[:90]} | {n} | {avg / 1e3:.3f} | {lo / 1e3:.3f} | {hi / 1e3:.3f} | "
                             f"{tot / 1e3:.1f}")
    con.close()
    return lines


def main(argv: list[str]) -> int:
    if len(argv) < 2:
        print(__doc__)
        return 2
    print("\n".join(summarise(argv[1], argv[2:])))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv))
