"""Per-kernel times of one engine step from a ``rocprofv3 --kernel-trace`` database.

    python -m macllm_infer_amd.utils.kernel_trace RESULTS.db [--first KERNEL] [--top N]

A step starts at the last launch of the kernel whose name contains ``--first`` (default: the
embedding kernel, the first launch of every forward pass) and runs to the end of the trace or,
with ``--last``, to the last launch of that kernel.  Prints launches, busy time (sum of kernel
durations), span (first start to last end) and the kernels by total time.
"""
from __future__ import annotations

import argparse
import sqlite3
from collections import defaultdict


def last_step(database: str, first: str, last: str | None):
    connection = sqlite3.connect(database)
    kernels = connection.execute("select name, start, end from kernels order by start").fetchall()
    starts = [index for index, row in enumerate(kernels) if first in row[0]]
    if not starts:
        raise SystemExit(f"no kernel whose name contains {first!r} in {database}")
    begin = starts[-1]
    end = len(kernels)
    if last is not None:
        ends = [index for index, row in enumerate(kernels) if last in row[0] and index >= begin]
        if ends:
            end = ends[-1] + 1
        else:                                   # the trace ends inside a step: take the one before
            begin = starts[-2]
            end = [index for index, row in enumerate(kernels) if last in row[0] and index >= begin][0] + 1
    return kernels[begin:end]


def main() -> None:
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    parser.add_argument("database")
    parser.add_argument("--first", default="embed_kernel")
    parser.add_argument("--last", default=None)
    parser.add_argument("--top", type=int, default=24)
    args = parser.parse_args()
    step = last_step(args.database, args.first, args.last)
    busy = sum(end - start for _, start, end in step)
    span = step[-1][2] - step[0][1]
    print(f"launches {len(step)}   busy {busy / 1e3:.1f} us   span {span / 1e3:.1f} us")
    totals = defaultdict(lambda: [0, 0])
    for name, start, end in step:
        totals[name][0] += 1
        totals[name][1] += end - start
    print(f"{'kernel':72s} {'calls':>5s} {'total us':>10s} {'avg us':>8s} {'share':>6s}")
    for name, (calls, total) in sorted(totals.items(), key=lambda item: -item[1][1])[:args.top]:
        print(f"{name[:72]:72s} {calls:5d} {total / 1e3:10.1f} {total / calls / 1e3:8.2f} {100.0 * total / busy:5.1f}%")


if __name__ == "__main__":
    main()
