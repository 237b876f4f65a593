#!/usr/bin/env python3
"""Per-kernel summary of a rocprofv3 run that wrote a rocpd database
(``rocprofv3 --kernel-trace --stats -d DIR -o NAME -- ...`` -> DIR/NAME_results.db).

    python scripts/rocpd_summary.py DB [--like PATTERN] [--top N]

Groups dispatches by kernel name and launch shape (workgroups per dimension)
and prints calls, mean and total time. ``--like`` (SQL LIKE pattern) restricts
the time window to the span between the first and the last dispatch of the
matching kernels, e.g. one model family's part of a run.
"""
import argparse
import sqlite3


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__,
                                 formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("db")
    ap.add_argument("--like", default="")
    ap.add_argument("--top", type=int, default=40)
    a = ap.parse_args()
    c = sqlite3.connect(a.db)
    where, args = "", ()
    if a.like:
        t0, t1 = c.execute("select min(start), max(end) from kernels where name like ?",
                           (a.like,)).fetchone()
        if t0 is None:
            print("no kernel matches", a.like)
            return 1
        where, args = "where start >= ? and end <= ?", (t0, t1)
    rows = c.execute(
        "select name, grid_x / workgroup_x, grid_y / workgroup_y, grid_z / workgroup_z, count(*), "
        f"avg(end - start) / 1e3, sum(end - start) / 1e3 from kernels {where} "
        "group by name, grid_x, grid_y, grid_z order by 7 desc", args).fetchall()
    total = sum(r[6] for r in rows)
    print(f"{len(rows)} (kernel, launch shape) groups, {total / 1e3:.2f} ms of kernel time")
    print(f"{'total us':>10} {'share':>6} {'calls':>6} {'mean us':>9}  workgroups      kernel")
    for r in rows[: a.top]:
        shape = f"({r[1]},{r[2]},{r[3]})"
        print(f"{r[6]:10.0f} {100 * r[6] / total:5.1f}% {r[4]:6d} {r[5]:9.1f}  {shape:<15} {r[0][:110]}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
