"""Per-kernel hardware counters of one engine step from ``rocprofv3 --pmc ... --output-format csv``.

    python -m macllm_infer_amd.utils.counter_summary COUNTERS.csv [MORE.csv ...] [--first KERNEL] [--last KERNEL]

Each file is the ``*_counter_collection.csv`` of one counter pass over the same program.  A step
starts at the last launch of the kernel whose name contains ``--first`` and ends at the last launch
(after it) of the kernel whose name contains ``--last``, or with the file.  Prints, per kernel, the
launches of the step and the sum of every counter over them.
"""
from __future__ import annotations

import argparse
import csv
from collections import OrderedDict, defaultdict


def last_step(path: str, first: str, last: str | None):
    """[(kernel name, {counter: value})] of the last step, in launch order."""
    dispatches: "OrderedDict[int, tuple]" = OrderedDict()
    with open(path, newline="") as handle:
        for row in csv.DictReader(handle):
            key = int(row["Dispatch_Id"])
            if key not in dispatches:
                dispatches[key] = (row["Kernel_Name"], {})
            dispatches[key][1][row["Counter_Name"]] = float(row["Counter_Value"])
    launches = [dispatches[key] for key in sorted(dispatches)]
    starts = [index for index, (name, _) in enumerate(launches) if first in name]
    if not starts:
        raise SystemExit(f"no kernel whose name contains {first!r} in {path}")
    for begin in reversed(starts):
        if last is None:
            return launches[begin:]
        ends = [index for index, (name, _) in enumerate(launches) if last in name and index >= begin]
        if ends:
            return launches[begin:ends[-1] + 1]
    raise SystemExit(f"no step from {first!r} to {last!r} in {path}")


def main() -> None:
    parser = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    parser.add_argument("files", nargs="+")
    parser.add_argument("--first", default="embed_kernel")
    parser.add_argument("--last", default=None)
    parser.add_argument("--top", type=int, default=20)
    args = parser.parse_args()
    calls: dict = {}
    sums: dict = defaultdict(lambda: defaultdict(float))
    counters: list = []
    for path in args.files:
        step = last_step(path, args.first, args.last)
        seen = defaultdict(int)
        for name, values in step:
            seen[name] += 1
            for counter, value in values.items():
                sums[name][counter] += value
                if counter not in counters:
                    counters.append(counter)
        for name, count in seen.items():
            calls[name] = count
    order = sorted(calls, key=lambda name: -sums[name].get(counters[0], 0.0))[:args.top]
    print(f"{'kernel':56s} {'calls':>5s} " + " ".join(f"{counter[:22]:>22s}" for counter in counters))
    for name in order:
        print(f"{name[:56]:56s} {calls[name]:5d} " + " ".join(f"{sums[name].get(counter, 0.0):22.1f}" for counter in counters))
    print(f"{'all kernels of the step':56s} {sum(calls.values()):5d} "
          + " ".join(f"{sum(sums[name].get(counter, 0.0) for name in calls):22.1f}" for counter in counters))


if __name__ == "__main__":
    main()
