"""Per-kernel totals of a rocprofv3 kernel trace.

    python profile_summary.py RESULTS.db [TOP] [--match TEXT] [--tail-ms MS]

reads the ``kernels`` view of the rocpd SQLite file that
``rocprofv3 --kernel-trace --stats -d DIR -o NAME -- <program>`` writes
(``DIR/NAME_results.db``) and prints calls, total, share, mean, min and max time per
kernel name, longest total first. ``--tail-ms MS`` keeps only the launches of the
last MS milliseconds of the trace (the timed steps of a benchmark, without its set-up).

    python profile_summary.py --counters COUNTERS.csv [--match TEXT]

reads the ``*_counter_collection.csv`` of ``rocprofv3 --pmc ... --output-format csv`` and
prints, per kernel name, the mean of each counter over the kernel's launches.
"""

from __future__ import annotations

import sqlite3
import sys


def summarise(path: str, top: int = 25, match: str | None = None, tail_ms: float | None = None) -> str:
    con = sqlite3.connect(path)
    since = 0
    if tail_ms is not None:
        since = con.execute("select max(end) from kernels").fetchone()[0] - int(tail_ms * 1e6)
    rows = con.execute("select name, count(*), sum(end - start), min(end - start), max(end - start) "
                       "from kernels where start >= ? group by name order by 3 desc", (since,)).fetchall()
    if match:
        rows = [r for r in rows if match in r[0]]
    total = sum(r[2] for r in rows) or 1
    out = [f"total kernel time {total / 1e6:.3f} ms over {sum(r[1] for r in rows)} launches",
           f"{'kernel':72s} {'calls':>7s} {'total ms':>10s} {'%':>6s} {'avg us':>9s} {'min us':>9s} {'max us':>9s}"]
    for name, calls, t, mn, mx in rows[:top]:
        out.append(f"{name[:72]:72s} {calls:7d} {t / 1e6:10.3f} {100 * t / total:6.2f} {t / calls / 1e3:9.1f} "
                   f"{mn / 1e3:9.1f} {mx / 1e3:9.1f}")
    return "\n".join(out)


def counters(path: str, match: str | None = None) -> str:
    import collections
    import csv

    total: dict = collections.defaultdict(lambda: collections.defaultdict(float))
    count: dict = collections.Counter()
    with open(path, newline="") as f:
        for row in csv.DictReader(f):
            name = row["Kernel_Name"]
            if match and match not in name:
                continue
            total[name][row["Counter_Name"]] += float(row["Counter_Value"])
            count[(name, row["Counter_Name"])] += 1
    out = []
    for name, vals in total.items():
        out.append(name[:100])
        for c, v in sorted(vals.items()):
            out.append(f"    {c:34s} {v / count[(name, c)]:18.1f}   (mean of {count[(name, c)]} launches)")
    return "\n".join(out)


def main(argv: list[str]) -> int:
    if not argv:
        print(__doc__)
        return 2
    match = None
    if "--match" in argv:
        i = argv.index("--match")
        match = argv[i + 1]
        del argv[i:i + 2]
    if "--counters" in argv:
        print(counters(argv[argv.index("--counters") + 1], match))
        return 0
    tail_ms = None
    if "--tail-ms" in argv:
        i = argv.index("--tail-ms")
        tail_ms = float(argv[i + 1])
        del argv[i:i + 2]
    print(summarise(argv[0], int(argv[1]) if len(argv) > 1 else 25, match, tail_ms))
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
