#!/usr/bin/env python3
"""Summarise a rocprofv3 (rocpd sqlite) kernel trace: per-kernel calls / total / avg / min / max (us).

    rocpd_stats.py results.db [top] [--grid PREFIX]

--grid PREFIX: only kernels whose name starts with PREFIX (e.g. stk_), one line per launch grid (threads), so that the shapes of a
run (prompt steps of several sizes, decode steps) stay apart."""
import re
import sqlite3
import sys


def short_name(name):
    short = name.replace("(anonymous namespace)::", "")
    short = re.sub(r"\(.*", "", short)
    return re.sub(r"^void ", "", short)


def by_grid(path, prefix, top):
    cur = sqlite3.connect(path).cursor()
    agg = {}
    for name, s, e, gx, gy, gz in cur.execute("select name, start, end, grid_x, grid_y, grid_z from kernels"):
        n = short_name(name)
        if not n.startswith(prefix):
            continue
        a = agg.setdefault((n, gx, gy, gz), [0, 0.0, 1e30])
        d = (e - s) / 1e3
        a[0] += 1
        a[1] += d
        a[2] = min(a[2], d)
    for k, a in sorted(agg.items(), key=lambda kv: -kv[1][1])[:top]:
        print(f"{k[0][:62]:62s} grid {k[1]:>7}x{k[2]:<4}x{k[3]:<3} calls {a[0]:5d} total {a[1]:10.1f} avg {a[1]/a[0]:8.2f} min {a[2]:8.2f}")


def main(path, top=40):
    db = sqlite3.connect(path)
    cur = db.cursor()
    cols = [r[1] for r in cur.execute("pragma table_info(kernels)")]
    name_col = "name" if "name" in cols else [c for c in cols if "name" in c][0]
    rows = cur.execute(f"select {name_col}, start, end from kernels").fetchall()
    agg = {}
    for name, s, e in rows:
        short = short_name(name)
        a = agg.setdefault(short, [0, 0.0, 1e30, 0.0])
        d = (e - s) / 1e3
        a[0] += 1
        a[1] += d
        a[2] = min(a[2], d)
        a[3] = max(a[3], d)
    tot = sum(a[1] for a in agg.values())
    print(f"{'kernel':70s} {'calls':>7s} {'total_us':>12s} {'avg_us':>9s} {'min_us':>9s} {'max_us':>9s} {'%':>6s}")
    for k, a in sorted(agg.items(), key=lambda kv: -kv[1][1])[:top]:
        print(f"{k[:70]:70s} {a[0]:7d} {a[1]:12.1f} {a[1]/a[0]:9.2f} {a[2]:9.2f} {a[3]:9.2f} {100*a[1]/tot:6.2f}")
    print(f"total kernel time {tot/1e3:.2f} ms over {len(rows)} dispatches")


if __name__ == "__main__":
    args = sys.argv[1:]
    prefix = None
    if "--grid" in args:
        i = args.index("--grid")
        prefix = args[i + 1]
        del args[i:i + 2]
    n = int(args[1]) if len(args) > 1 else 40
    if prefix is not None:
        by_grid(args[0], prefix, n)
    else:
        main(args[0], n)
