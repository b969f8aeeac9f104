"""What a kernel trace says about a run: time by kernel, and how much of the wall time no kernel ran.

Reads the results database that ``rocprofv3 --kernel-trace`` writes (SQLite; its ``kernels`` view has one row a
launch with ``name``, ``start`` and ``end`` in nanoseconds, and the grid's size) and prints text, short enough
to keep beside the code:

    python3 -m tie_amd.bench.kernel_trace RESULTS.db                 # totals by kernel
    python3 -m tie_amd.bench.kernel_trace RESULTS.db --steps 8       # the last 8 decode steps, a step's average
    python3 -m tie_amd.bench.kernel_trace RESULTS.db --window 3.4    # busy share of the run's last 3.4 seconds

A decode step starts at the embedding kernel (``--step-starts-at`` names another). The busy share counts a
moment as busy when at least one kernel runs; the gaps between kernels are what the host, the launches and the
reads of results cost. The counterpart in the reference is the per-phase timing of its bench report
(src/bench/report.h:29-36); a kernel-level view has none there.
"""
from __future__ import annotations

import argparse
import collections
import re
import sqlite3
import sys
from typing import List, Sequence, Tuple

Launch = Tuple[str, int, int, int]        # name, start ns, end ns, threads of the grid


def short_name(name: str, width: int = 72) -> str:
    name = re.sub(r"^void ", "", name)
    return re.sub(r"\(.*", "", name)[:width]


def read_launches(path: str) -> List[Launch]:
    db = sqlite3.connect(path)
    columns = [row[1] for row in db.execute("pragma table_info(kernels)")]
    if not columns:
        raise SystemExit(f"{path}: no 'kernels' view (was the run traced with --kernel-trace?)")
    grid = "grid_x * grid_y * grid_z" if {"grid_x", "grid_y", "grid_z"} <= set(columns) else "0"
    return [(n, s, e, g) for n, s, e, g in db.execute(f"select name, start, end, {grid} from kernels order by start")]


def totals(launches: Sequence[Launch], by_grid: bool = False, top: int = 25) -> str:
    agg = collections.OrderedDict()
    for name, start, end, grid in launches:
        entry = agg.setdefault((short_name(name), grid if by_grid else 0), [0, 0])
        entry[0] += 1
        entry[1] += end - start
    total = sum(v[1] for v in agg.values()) or 1
    lines = [f"{'kernel':72s} {'calls':>7s} {'total ms':>10s} {'avg us':>9s} {'%':>6s}"]
    for (name, grid), (calls, ns) in sorted(agg.items(), key=lambda kv: -kv[1][1])[:top]:
        label = f"{name} [{grid} threads]" if by_grid else name
        lines.append(f"{label[:72]:72s} {calls:7d} {ns / 1e6:10.3f} {ns / calls / 1e3:9.2f} {100 * ns / total:6.1f}")
    lines.append(f"kernel time {total / 1e6:.1f} ms over a span of {(launches[-1][2] - launches[0][1]) / 1e6:.1f} ms")
    return "\n".join(lines)


def last_steps(launches: Sequence[Launch], steps: int, starts_at: str, by_grid: bool = False) -> str:
    starts = [i for i, launch in enumerate(launches) if starts_at in launch[0]][-steps - 1:]
    if len(starts) < 2:
        raise SystemExit(f"fewer than two launches of a kernel named like '{starts_at}'")
    n = len(starts) - 1
    agg = collections.OrderedDict()
    span = busy = 0
    for a, b in zip(starts[:-1], starts[1:]):
        step = launches[a:b]
        span += step[-1][2] - step[0][1]
        for name, start, end, grid in step:
            entry = agg.setdefault((short_name(name), grid if by_grid else 0), [0, 0])
            entry[0] += 1
            entry[1] += end - start
            busy += end - start
    period = (launches[starts[-1]][1] - launches[starts[0]][1]) / n
    lines = [f"{n} steps: kernel span {span / n / 1e3:.1f} us/step, kernel busy {busy / n / 1e3:.1f} us/step, "
             f"step period {period / 1e3:.1f} us",
             f"{'kernel':72s} {'calls/step':>10s} {'us/call':>9s} {'us/step':>9s} {'%busy':>6s}"]
    for (name, grid), (calls, ns) in sorted(agg.items(), key=lambda kv: -kv[1][1]):
        label = f"{name} [{grid} threads]" if by_grid else name
        lines.append(f"{label[:72]:72s} {calls / n:10.1f} {ns / calls / 1e3:9.2f} {ns / n / 1e3:9.1f} {100 * ns / busy:6.1f}")
    return "\n".join(lines)


def busy_share(launches: Sequence[Launch], window_s: float) -> str:
    """Over the last ``window_s`` seconds before the last kernel's end (the timed part of a run that warms up first)."""
    t_end = launches[-1][2]
    t0 = t_end - int(window_s * 1e9)
    busy, last_end, gaps = 0, t0, []
    for _, start, end, _ in launches:
        if end <= t0:
            continue
        start = max(start, t0)
        if start > last_end:
            gaps.append(start - last_end)
        busy += max(0, end - max(start, last_end))
        last_end = max(last_end, end)

    def total(lo, hi):
        chosen = [g for g in gaps if lo < g <= hi]
        return len(chosen), sum(chosen) / 1e9

    long_n, long_s = total(1e5, float("inf"))
    mid_n, mid_s = total(2e4, 1e5)
    short_n, short_s = total(0, 2e4)
    return (f"last {window_s:.2f} s: a kernel runs during {busy / 1e9:.3f} s = {busy / (window_s * 1e9):.3f} of it; "
            f"gaps over 100 us: {long_n} totalling {long_s:.3f} s; 20 to 100 us: {mid_n} totalling {mid_s:.3f} s; "
            f"shorter: {short_n} totalling {short_s:.3f} s")


def main(argv=None) -> int:
    parser = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    parser.add_argument("database", help="the results database of rocprofv3 --kernel-trace")
    parser.add_argument("--steps", type=int, default=0, help="average over the last N decode steps instead of the whole run")
    parser.add_argument("--step-starts-at", default="embed_kernel", help="part of the name of a step's first kernel")
    parser.add_argument("--window", type=float, default=0.0, help="also: the busy share of the last S seconds")
    parser.add_argument("--by-grid", action="store_true", help="tell launches of one kernel apart by their grid's size")
    parser.add_argument("--top", type=int, default=25, help="kernels listed in the totals")
    args = parser.parse_args(argv)
    launches = read_launches(args.database)
    if not launches:
        raise SystemExit("the trace holds no kernel")
    if args.steps > 0:
        print(last_steps(launches, args.steps, args.step_starts_at, args.by_grid))
    else:
        print(totals(launches, args.by_grid, args.top))
    if args.window > 0:
        print(busy_share(launches, args.window))
    return 0


if __name__ == "__main__":
    sys.exit(main())
