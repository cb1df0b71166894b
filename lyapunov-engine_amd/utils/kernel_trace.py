"""Summarise a rocprofv3 kernel trace per engine step.

    rocprofv3 --kernel-trace -d OUT -o NAME -- python3 bench.py ...
    python -m lyapunov_engine_amd.utils.kernel_trace OUT/NAME_results.db [--step N]
    python -m lyapunov_engine_amd.utils.kernel_trace OUT/NAME_results.db --all     (any program's kernels)

A step starts at the embedding kernel.  For the chosen step (default: the third
from the end, a steady decode step of the bench) it prints the GPU time from the
first kernel's start to the last kernel's end, the idle time until the next
step's first kernel (host work), and per kernel and launch shape the number of
launches and their total and mean duration.

The reference has no tracing of its own; its benches time with CUDA events
(benchmarks/bench_kernels.py:7-27).
"""
from __future__ import annotations

import argparse
import collections
import sqlite3


def short(name: str) -> str:
    for mark in ("lyp::", "_ZN3lyp"):
        i = name.find(mark)
        if i >= 0:
            name = name[i:]
            break
    return name[:72]


def summarise(db: str, step: int) -> str:
    con = sqlite3.connect(db)
    rows = con.execute(
        "select name, start, end, grid_x, grid_y, grid_z, workgroup_x from kernels order by start").fetchall()
    starts = [i for i, r in enumerate(rows) if "embedding_kernel" in r[0]]
    if len(starts) < 2:
        raise SystemExit("the trace holds fewer than two engine steps")
    a = starts[step]
    b = starts[step + 1] if step + 1 < len(starts) and step != -1 else len(rows)
    chunk = rows[a:b]
    lines = [f"step {step} of {len(starts)}: {len(chunk)} kernels, "
             f"{(chunk[-1][2] - chunk[0][1]) / 1e3:.1f} us from first start to last end"
             + (f", {(rows[b][1] - chunk[-1][2]) / 1e3:.1f} us idle before the next step" if b < len(rows) else "")]
    agg: dict = collections.OrderedDict()
    for name, t0, t1, gx, gy, gz, wg in chunk:
        key = (short(name), gx // max(wg, 1), gy, gz, wg)
        n, t = agg.get(key, (0, 0.0))
        agg[key] = (n + 1, t + (t1 - t0) / 1e3)
    lines.append(f"{'total us':>10} {'calls':>6} {'mean us':>9}  workgroups x threads   kernel")
    for (name, gx, gy, gz, wg), (n, t) in sorted(agg.items(), key=lambda kv: -kv[1][1]):
        lines.append(f"{t:10.1f} {n:6d} {t / n:9.2f}  ({gx},{gy},{gz}) x {wg:<5d}  {name}")
    return "\n".join(lines)


def summarise_all(db: str, skip: int) -> str:
    """Every kernel of the trace by name and launch shape: launches, median and mean duration,
    leaving out each kind's first ``skip`` launches (a program's warm-up calls)."""
    con = sqlite3.connect(db)
    rows = con.execute(
        "select name, start, end, grid_x, grid_y, grid_z, workgroup_x from kernels order by start").fetchall()
    agg: dict = collections.OrderedDict()
    for name, t0, t1, gx, gy, gz, wg in rows:
        agg.setdefault((short(name), gx // max(wg, 1), gy, gz, wg), []).append((t1 - t0) / 1e3)
    lines = [f"{'calls':>6} {'median us':>10} {'mean us':>9}  workgroups x threads   kernel"]
    for (name, gx, gy, gz, wg), ts in sorted(agg.items(), key=lambda kv: -sum(kv[1])):
        ts = sorted(ts[skip:] or ts)
        lines.append(f"{len(ts):6d} {ts[len(ts) // 2]:10.2f} {sum(ts) / len(ts):9.2f}  ({gx},{gy},{gz}) x {wg:<5d}  {name}")
    return "\n".join(lines)


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("db", help="rocprofv3's NAME_results.db")
    ap.add_argument("--step", type=int, default=-3, help="which step (negative: from the end)")
    ap.add_argument("--all", action="store_true", help="every kernel of the trace by name and shape (a program that "
                    "is no engine: kernel_bench), not one engine step")
    ap.add_argument("--skip", type=int, default=2, help="with --all: launches of every kind left out as warm-up")
    args = ap.parse_args()
    print(summarise_all(args.db, args.skip) if args.all else summarise(args.db, args.step))


if __name__ == "__main__":
    main()
