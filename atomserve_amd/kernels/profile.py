"""Summarise a rocprofv3 kernel trace (`*_results.db`) as text: time per kernel, and
per decode step when the steps can be told apart by a marker kernel; or, for a run with
`--pmc`, the counters of the kernels whose names contain a given text.

    python -m atomserve_amd.kernels.profile RESULTS.db [--steps N [--marker NAME | --begin NAME [--having NAME]]] [--top K]
    python -m atomserve_amd.kernels.profile RESULTS.db --counters NAME_PART
"""

import argparse
import sqlite3


def summarise(db: str, steps: int = 0, marker: str = "sample_", top: int = 20, begin: str = "", having: str = "") -> str:
    rows = sqlite3.connect(db).execute("select name, start, end from kernels order by start").fetchall()
    lines = []
    if steps and begin:  # the last `steps` steps of the trace, each from a kernel named *begin* to the next such
        marks = [i for i, r in enumerate(rows) if begin in r[0]]
        cuts = [rows[a:b] for a, b in zip(marks, marks[1:] + [len(rows)])]
        cuts = [c for c in cuts if any(having in r[0] for r in c)]
        if len(cuts) < steps:
            raise SystemExit(f"only {len(cuts)} steps from {begin!r} with {having!r}; cannot cut {steps}")
        cuts = cuts[-steps:]
        span = sum(c[-1][2] - c[0][1] for c in cuts)
        rows, marker = [r for c in cuts for r in c], f"from {begin}" + (f"* with {having}" if having else "")
    elif steps:
        marks = [i for i, r in enumerate(rows) if marker in r[0]]
        if len(marks) <= steps:
            raise SystemExit(f"only {len(marks)} launches of {marker!r}; cannot cut {steps} steps")
        span = rows[marks[-1]][2] - rows[marks[-steps - 1]][2]
        rows = rows[marks[-steps - 1] + 1 : marks[-1] + 1]
    agg: dict = {}
    for name, start, end in rows:
        a = agg.setdefault(name, [0, 0])
        a[0] += 1
        a[1] += end - start
    total = sum(a[1] for a in agg.values())
    div = steps or 1
    cut = marker if begin else "at " + marker
    ends = "a step's first kernel to its last" if begin else "step to step"
    unit = "per step" if steps else "in all"
    lines.append(f"{len(rows) / div:.0f} launches, {total / div / 1e3:.1f} us of kernel time {unit}"
                 + (f" (last {steps} steps, cut {cut}*; {span / div / 1e3:.1f} us from {ends})" if steps else ""))  # fmt: skip
    lines.append(f"{'kernel':64s} {'launches':>9s} {'us ' + unit:>12s} {'avg us':>9s} {'share':>6s}")
    for name, (count, t) in sorted(agg.items(), key=lambda kv: -kv[1][1])[:top]:
        lines.append(f"{name[:64]:64s} {count / div:9.1f} {t / div / 1e3:12.1f} {t / count / 1e3:9.2f} {100 * t / total:5.1f}%")
    return "\n".join(lines)


def counters(db: str, name_part: str) -> str:
    """Mean value per dispatch of every collected counter, for each kernel whose name contains
    `name_part` (counters are sums over the chip; SQ_*_CYCLES of waves count in units of four)."""
    rows = sqlite3.connect(db).execute(
        "select kernel_name, counter_name, sum(value), count(distinct dispatch_id), avg(end - start) "
        "from counters_collection where kernel_name like ? group by 1, 2 order by 1, 2", (f"%{name_part}%",)
    ).fetchall()  # fmt: skip
    lines, last = [], None
    for kernel, counter, total, dispatches, ns in rows:
        if kernel != last:
            lines.append(f"{kernel[:100]}  ({dispatches} dispatches, {ns / 1e3:.1f} us each while counting)")
            last = kernel
        lines.append(f"    {counter:40s} {total / max(dispatches, 1):16.4g}")
    return "\n".join(lines) if lines else f"no counters for kernels named *{name_part}*"


if __name__ == "__main__":
    p = argparse.ArgumentParser()
    p.add_argument("db")
    p.add_argument("--steps", type=int, default=0)
    p.add_argument("--marker", default="sample_", help="part of the name of the kernel that ends a step")
    p.add_argument("--begin", default="", help="part of the name of the kernel that begins a step (instead of --marker)")
    p.add_argument("--having", default="", help="with --begin: only steps that launch a kernel of this name")
    p.add_argument("--top", type=int, default=20)
    p.add_argument("--counters", default="", help="part of a kernel name: print its counters instead")
    a = p.parse_args()
    print(counters(a.db, a.counters) if a.counters else summarise(a.db, a.steps, a.marker, a.top, a.begin, a.having))
