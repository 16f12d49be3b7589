"""Summaries of a ``rocprofv3 --kernel-trace`` CSV: per-kernel time, the span
of a region and the share of it in which at least one kernel ran.

``python -m flex_shard_amd.trace_summary TRACE.csv [--step-kernel NAME
--per-step N --skip-steps K]``

A trace has no marker for "the timed steps", so the region is named through a
kernel that runs a known number of times per step (``--step-kernel``, matched
as a substring of the kernel name; ``--per-step`` launches per step): the
first ``--skip-steps`` steps are dropped and the region runs from the end of
the last dropped step's last such launch to the end of the trace's last such
launch.  Without ``--step-kernel`` the whole trace is the region.
``--kernel NAME --first I --count N`` prints instead the duration statistics
of dispatches I .. I+N-1 (start order) of one kernel, for a benchmark whose
sections issue a known number of launches each.  ``--counters`` reads a
``rocprofv3 --pmc`` ``*_counter_collection.csv`` instead and prints the average
reading per dispatch of every kernel and counter.

Figures: ``span`` = last end - first start inside the region; ``busy`` = the
length of the union of all kernel intervals (kernels on different streams
overlap, so the sum of kernel times can exceed the span); per kernel: launches,
total, average, share of the summed kernel time.  Kernel names are shortened
to the function name (template and argument lists dropped).
"""

from __future__ import annotations

import argparse
import csv
import re
import sys
from collections import defaultdict


def short_name(name: str) -> str:
    """``void ns::(anonymous namespace)::kernel<...>(args)`` -> ``kernel<...>``
    with nested template arguments and the argument list dropped."""
    name = re.sub(r"^void\s+", "", name.strip())
    # torch's generic elementwise / reduction kernels are told apart by their functor
    functor = re.search(r"(\w*Functor\w*|\w+_functor|\w*copy_kernel\w*|normal_kernel)", name)
    if functor and re.match(r"at::native::", name):
        generic = re.match(r"at::native::(?:\(anonymous namespace\)::)?(\w+)", name)
        return f"{generic.group(1) if generic else 'kernel'}[{functor.group(1)}]"
    depth, cut = 0, len(name)
    for index, ch in enumerate(name):  # cut the argument list: the first '(' outside <...> that is not "(anonymous"
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        elif ch == "(" and depth == 0 and not name.startswith("(anonymous", index):
            cut = index
            break
    name = name[:cut]
    head, sep, tail = name.partition("<")
    head = head.split("::")[-1]
    if not sep:
        return head
    tail = tail.rsplit(">", 1)[0]
    if len(tail) > 24 or "<" in tail:
        # keep the leading template arguments that are plain tokens (ints, bools, short type names)
        plain = []
        for token in tail.split(","):
            token = token.strip()
            if re.fullmatch(r"[\w:]{1,16}", token):
                plain.append(token.split("::")[-1])
            else:
                break
        tail = ", ".join(plain) + (", ..." if plain else "...")
    return f"{head}<{tail}>"


def read_trace(path: str) -> list[tuple[str, int, int]]:
    """(kernel name, start ns, end ns) of every dispatch, in start order."""
    rows = []
    with open(path, newline="") as fh:
        for row in csv.DictReader(fh):
            rows.append((row["Kernel_Name"], int(row["Start_Timestamp"]), int(row["End_Timestamp"])))
    rows.sort(key=lambda r: r[1])
    return rows


def select_region(rows, step_kernel: str | None, per_step: int, skip_steps: int):
    """The dispatches of the region and the number of steps it holds."""
    if not step_kernel:
        return rows, None
    marks = [end for name, _, end in rows if step_kernel in name]
    if per_step <= 0 or len(marks) % per_step:
        raise SystemExit(f"{len(marks)} launches of {step_kernel!r} are not a multiple of --per-step {per_step}")
    steps = len(marks) // per_step
    if skip_steps >= steps:
        raise SystemExit(f"the trace holds {steps} steps; cannot skip {skip_steps}")
    begin = marks[skip_steps * per_step - 1] if skip_steps else rows[0][1]
    end = marks[-1]
    return [r for r in rows if r[1] >= begin and r[2] <= end], steps - skip_steps


def union_length(intervals) -> int:
    total, current_start, current_end = 0, None, None
    for start, end in sorted(intervals):
        if current_end is None or start > current_end:
            if current_end is not None:
                total += current_end - current_start
            current_start, current_end = start, end
        else:
            current_end = max(current_end, end)
    if current_end is not None:
        total += current_end - current_start
    return total


def summarize(rows, steps: int | None) -> str:
    if not rows:
        return "no dispatches in the region"
    span = max(r[2] for r in rows) - min(r[1] for r in rows)
    busy = union_length((r[1], r[2]) for r in rows)
    per_kernel = defaultdict(lambda: [0, 0])
    for name, start, end in rows:
        entry = per_kernel[short_name(name)]
        entry[0] += 1
        entry[1] += end - start
    summed = sum(v[1] for v in per_kernel.values())
    per = f" ({steps} steps)" if steps else ""
    lines = [
        f"region{per}: span {span / 1e6:.3f} ms, busy (union of kernel intervals) {busy / 1e6:.3f} ms = "
        f"{100 * busy / span:.1f} % of the span, summed kernel time {summed / 1e6:.3f} ms "
        f"({summed / span:.2f} x the span: kernels on different streams overlap), {len(rows)} dispatches",
    ]
    if steps:
        lines.append(
            f"per step: span {span / steps / 1e6:.3f} ms, busy {busy / steps / 1e6:.3f} ms, summed kernel time "
            f"{summed / steps / 1e6:.3f} ms, idle {(span - busy) / steps / 1e3:.1f} us"
        )
    lines.append("")
    lines.append(f"{'kernel':<64} {'calls':>6} {'total ms':>10} {'avg us':>10} {'share':>7}")
    for name, (calls, total) in sorted(per_kernel.items(), key=lambda kv: -kv[1][1]):
        lines.append(f"{name[:64]:<64} {calls:>6} {total / 1e6:>10.3f} {total / calls / 1e3:>10.1f} {100 * total / summed:>6.1f}%")
    return "\n".join(lines)


def kernel_slice(rows, kernel: str, first: int, count: int) -> str:
    """Duration statistics of dispatches [first, first + count) (0-based, in
    start order) of the kernel whose name contains ``kernel``."""
    mine = [(start, end) for name, start, end in rows if kernel in name]
    chosen = mine[first : first + count if count else None]
    if not chosen:
        return f"{kernel}: {len(mine)} dispatches in the trace, none in the slice"
    durations = sorted((end - start) / 1e3 for start, end in chosen)
    span = chosen[-1][1] - chosen[0][0]
    return (
        f"{kernel}: dispatches {first}..{first + len(chosen) - 1} of {len(mine)}: avg {sum(durations) / len(durations):.2f} us, "
        f"median {durations[len(durations) // 2]:.2f}, min {durations[0]:.2f}, max {durations[-1]:.2f}; "
        f"first start to last end {span / 1e3:.1f} us = {span / 1e3 / len(chosen):.2f} us per dispatch"
    )


def counters_summary(path: str) -> str:
    """Per kernel and counter of a ``rocprofv3 --pmc`` CSV
    (``*_counter_collection.csv``): dispatches and the average reading per
    dispatch (a counter's rows of one dispatch, one per sampled instance, are
    added first)."""
    per_dispatch: dict[tuple[str, str, str], float] = defaultdict(float)
    with open(path, newline="") as fh:
        for row in csv.DictReader(fh):
            key = (short_name(row["Kernel_Name"]) + f" (grid {row['Grid_Size']})", row["Counter_Name"], row["Dispatch_Id"])
            per_dispatch[key] += float(row["Counter_Value"])
    totals: dict[tuple[str, str], list[float]] = defaultdict(list)
    for (kernel, counter, _), value in per_dispatch.items():
        totals[(kernel, counter)].append(value)
    lines = [f"{'kernel (grid size in threads)':<72} {'counter':<28} {'dispatches':>10} {'average':>16}"]
    for (kernel, counter), values in sorted(totals.items()):
        lines.append(f"{kernel[:72]:<72} {counter:<28} {len(values):>10} {sum(values) / len(values):>16.1f}")
    return "\n".join(lines)


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("trace", help="rocprofv3 *_kernel_trace.csv")
    ap.add_argument("--step-kernel", help="substring of a kernel name that runs --per-step times per step")
    ap.add_argument("--per-step", type=int, default=1)
    ap.add_argument("--skip-steps", type=int, default=0)
    ap.add_argument("--kernel", help="instead of the region summary: statistics of a slice of this kernel's dispatches")
    ap.add_argument("--first", type=int, default=0, help="with --kernel: index of the slice's first dispatch")
    ap.add_argument("--count", type=int, default=0, help="with --kernel: dispatches in the slice (0 = to the end)")
    ap.add_argument("--counters", action="store_true", help="the file is a --pmc counter_collection.csv: average readings")
    args = ap.parse_args(argv)
    if args.counters:
        sys.stdout.write(counters_summary(args.trace) + "\n")
        return
    trace = read_trace(args.trace)
    if args.kernel:
        sys.stdout.write(kernel_slice(trace, args.kernel, args.first, args.count) + "\n")
        return
    rows, steps = select_region(trace, args.step_kernel, args.per_step, args.skip_steps)
    sys.stdout.write(summarize(rows, steps) + "\n")


if __name__ == "__main__":
    main()
