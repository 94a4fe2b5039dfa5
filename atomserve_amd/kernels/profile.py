"""Summarise a rocprofv3 kernel trace (`*_results.db`) as text: time per kernel, and
per decode step when the steps can be told apart by a marker kernel.

    python -m atomserve_amd.kernels.profile RESULTS.db [--steps N --marker NAME] [--top K]
"""

import argparse
import sqlite3


def summarise(db: str, steps: int = 0, marker: str = "sample_kernel", top: int = 20) -> str:
    rows = sqlite3.connect(db).execute("select name, start, end from kernels order by start").fetchall()
    lines = []
    if steps:
        marks = [i for i, r in enumerate(rows) if marker in r[0]]
        if len(marks) <= steps:
            raise SystemExit(f"only {len(marks)} launches of {marker!r}; cannot cut {steps} steps")
        rows = rows[marks[-steps - 1] + 1 : marks[-1] + 1]
    agg: dict = {}
    for name, start, end in rows:
        a = agg.setdefault(name, [0, 0])
        a[0] += 1
        a[1] += end - start
    total = sum(a[1] for a in agg.values())
    div = steps or 1
    unit = "per step" if steps else "in all"
    lines.append(f"{len(rows) / div:.0f} launches, {total / div / 1e3:.1f} us of kernel time {unit}"
                 + (f" (last {steps} steps, cut at {marker})" if steps else ""))  # fmt: skip
    lines.append(f"{'kernel':64s} {'launches':>9s} {'us ' + unit:>12s} {'avg us':>9s} {'share':>6s}")
    for name, (count, t) in sorted(agg.items(), key=lambda kv: -kv[1][1])[:top]:
        lines.append(f"{name[:64]:64s} {count / div:9.1f} {t / div / 1e3:12.1f} {t / count / 1e3:9.2f} {100 * t / total:5.1f}%")
    return "\n".join(lines)


if __name__ == "__main__":
    p = argparse.ArgumentParser()
    p.add_argument("db")
    p.add_argument("--steps", type=int, default=0)
    p.add_argument("--marker", default="sample_kernel")
    p.add_argument("--top", type=int, default=20)
    a = p.parse_args()
    print(summarise(a.db, a.steps, a.marker, a.top))
