"""Per-kernel times of one engine step from a ``rocprofv3 --kernel-trace`` database, and, given the
model's sizes, what each group of kernels has to move and compute against the time it took.

    python -m macllm_infer_amd.utils.kernel_trace RESULTS.db [--first KERNEL] [--last KERNEL] [--top N]
        [--config CONFIG.json (--batch B --context C | --prefill T) [--dtype bf16|f32]] [--timeline FROM:TO]

A step starts at the last launch of the kernel whose name contains ``--first`` (default: the
embedding kernel, the first launch of every forward pass) and runs to the end of the trace or,
with ``--last``, to the last launch of that kernel.  Prints launches, busy time (sum of kernel
durations), span (first start to last end) and the kernels by total time.  With ``--config`` (a
config.json of the model that ran) and the step's shape it adds, per group of kernels: the bytes
the group has to read and write, its flops, the rates these make with the group's busy time, and
their fractions of the published peaks (8 TB/s; 2.5 PFLOP/s bf16, 157.3 TFLOP/s float32).
``--timeline FROM:TO`` lists launches FROM to TO of the step one by one (start after the first of them,
duration, the time since the latest end of everything before it): which kernels of a layer run side
by side on two streams, and where the GPU waits.
"""
from __future__ import annotations

import argparse
import json
import sqlite3
from collections import defaultdict

from . import costs


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


def roofline_table(step, spec, batch, context, prefill, dtype: str) -> None:
    element = 2 if dtype == "bf16" else 4
    if prefill:
        model, groups = costs.prefill_costs(spec, prefill, element), costs.PREFILL_GROUPS
    else:
        model, groups = costs.decode_step_costs(spec, batch, context, element), costs.DECODE_GROUPS
    busy = defaultdict(float)
    calls = defaultdict(int)
    for name, _, _ in step:
        calls[name] += 1
    for name, start, end in step:
        busy[costs.group_of(name, groups, calls[name]) or "(other kernels)"] += (end - start) * 1e-9
    print()
    print(f"{'group of kernels':44s} {'busy us':>9s} {'read MB':>9s} {'write MB':>9s} {'GB/s':>8s} {'of 8 TB/s':>9s} "
          f"{'GFLOP':>9s} {'TFLOP/s':>8s} {'of peak':>8s}")
    for name, seconds in sorted(busy.items(), key=lambda item: -item[1]):
        cost = costs.merged(model, name)
        moved = cost.read + cost.written
        if moved == 0 and cost.flops == 0:
            print(f"{name[:44]:44s} {seconds * 1e6:9.1f}")
            continue
        print(f"{name[:44]:44s} {seconds * 1e6:9.1f} {cost.read / 1e6:9.1f} {cost.written / 1e6:9.1f} "
              f"{moved / seconds / 1e9:8.0f} {moved / seconds / costs.PEAK_HBM_BYTES:9.3f} {cost.flops / 1e9:9.1f} "
              f"{cost.flops / seconds / 1e12:8.1f} {cost.flops / seconds / costs.PEAK_FLOPS[dtype]:8.4f}")
    whole = costs.total(model)
    seconds = sum(busy.values())
    print(f"{'the step (all kernels, busy time)':44s} {seconds * 1e6:9.1f} {whole.read / 1e6:9.1f} {whole.written / 1e6:9.1f} "
          f"{(whole.read + whole.written) / seconds / 1e9:8.0f} {(whole.read + whole.written) / seconds / costs.PEAK_HBM_BYTES:9.3f} "
          f"{whole.flops / 1e9:9.1f} {whole.flops / seconds / 1e12:8.1f} {whole.flops / seconds / costs.PEAK_FLOPS[dtype]:8.4f}")


def main() -> None:
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    parser.add_argument("database")
    parser.add_argument("--first", default="embed_kernel")
    parser.add_argument("--last", default=None)
    parser.add_argument("--top", type=int, default=24)
    parser.add_argument("--config", default=None, help="config.json of the model that ran: adds bytes, flops and fractions")
    parser.add_argument("--batch", type=int, default=0, help="requests of the decode step")
    parser.add_argument("--context", type=float, default=0, help="tokens each request of the decode step holds")
    parser.add_argument("--prefill", type=int, default=0, help="tokens of the prompt step (instead of --batch/--context)")
    parser.add_argument("--dtype", default="bf16", choices=["bf16", "f32"])
    parser.add_argument("--timeline", default=None, help="FROM:TO, launches of the step to list one by one")
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
    if args.timeline:
        low, high = (int(value) for value in args.timeline.split(":"))
        stretch = step[low:high]
        print()
        print(f"{'launch':>6s} {'start us':>9s} {'us':>8s} {'idle before':>11s}  kernel")
        latest = None
        for index, (name, start, end) in enumerate(stretch, low):
            idle = "" if latest is None else f"{(start - latest) / 1e3:11.2f}"
            print(f"{index:6d} {(start - stretch[0][1]) / 1e3:9.2f} {(end - start) / 1e3:8.2f} {idle:>11s}  {name[:60]}")
            latest = end if latest is None else max(latest, end)
    if args.config:
        from ..config.registry import config_from_dict
        with open(args.config) as handle:
            spec = config_from_dict(json.load(handle)).to_model_spec()
        if not args.prefill and not (args.batch and args.context):
            raise SystemExit("--config needs the step's shape: --batch and --context, or --prefill")
        roofline_table(step, spec, args.batch, args.context, args.prefill, args.dtype)


if __name__ == "__main__":
    main()
