#!/usr/bin/env python3
"""Condenses rocprofv3 CSV output into the short tables kept under profiles/.

    python -m tiny-cnn_amd.profsum kernels  <dir>            # --kernel-trace --stats run
    python -m tiny-cnn_amd.profsum counters <dir> [<dir>..]  # --pmc runs (one counter set per dir)
    python -m tiny-cnn_amd.profsum tags <dir> [<dir>..] --sequence seq.json [--merge profiles/hbm_traffic.json]

`tags` reads the same traces kernel tag by kernel tag. bench.py's per-kernel pass runs the
workload's steps eagerly with a mark in front of each (three launches of the fill kernel on one
small buffer) and, with --sequence-out, writes the tags of one step's launches in dispatch order.
Here the marks are found in the trace, the dispatches between two marks are matched one to one
with that sequence, and durations (kernel-trace directories) and counters (--pmc directories)
are averaged per tag: two tags that share a kernel symbol and grid (forward and dX of a
stride-1 convolution) get rows of their own. --merge writes the scaled FETCH_SIZE / WRITE_SIZE
bytes per launch into that JSON file under "workloads" / <workload> / <tag>.

`kernels` prints, per kernel symbol and grid size, launches and average/min/max duration from
`*_kernel_trace.csv` (kernel templates are launched at several problem shapes; the grid size
tells them apart). `counters` prints, per kernel symbol and grid size, the mean of every
counter in `*_counter_collection.csv`; with FETCH_SIZE / WRITE_SIZE present it also scales
them to bytes by what the same counters read for `copy_kernel`, the dispatch of known size
(it reads and writes `--copy-mib` MiB each).
"""
import argparse
import collections
import csv
import glob
import os
import re
import sys


def short_name(name):
    """`void tdh::x_kernel<5, 5>(...)` -> `x_kernel<5, 5>` with operand namespaces dropped."""
    name = re.sub(r"\(anonymous namespace\)::", "", name)
    name = re.sub(r"^void\s+", "", name).replace("tdh::", "")
    depth, out = 0, []
    for ch in name:  # cut the argument list: the first '(' outside template brackets
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        elif ch == "(" and depth == 0:
            break
        out.append(ch)
    return "".join(out).strip()


def find(dirname, suffix):
    hits = sorted(glob.glob(os.path.join(dirname, "**", "*" + suffix), recursive=True))
    if not hits:
        raise SystemExit(f"no *{suffix} under {dirname}")
    return hits


def kernels(dirname, top):
    """One row per kernel symbol and grid size. A replayed train step runs its weight-gradient
    kernels beside the main chain, and a kernel that shares the device takes longer than the
    same kernel alone; the "alone" columns average only the dispatches that overlap no other
    dispatch in time (the per-kernel pass of bench.py launches every kernel that way)."""
    disp = []
    for path in find(dirname, "_kernel_trace.csv"):
        with open(path, newline="") as f:
            for r in csv.DictReader(f):
                if "Grid_Size" in r:
                    grid = int(r["Grid_Size"])
                else:
                    grid = int(r["Grid_Size_X"]) * int(r["Grid_Size_Y"]) * int(r["Grid_Size_Z"])
                disp.append((int(r["Start_Timestamp"]), int(r["End_Timestamp"]),
                             (short_name(r["Kernel_Name"]), grid)))
    disp.sort()
    rows, alone = collections.defaultdict(list), collections.defaultdict(list)
    latest_end = 0  # of all earlier dispatches
    for k, (start, end, key) in enumerate(disp):
        rows[key].append(end - start)
        overlaps = start < latest_end or (k + 1 < len(disp) and disp[k + 1][0] < end)
        if not overlaps:
            alone[key].append(end - start)
        latest_end = max(latest_end, end)
    total = sum(sum(v) for v in rows.values())
    print("| kernel | grid (work-items) | launches | avg us | min us | max us | % of GPU time | alone: launches | alone: avg us |")
    print("|---|---:|---:|---:|---:|---:|---:|---:|---:|")
    order = sorted(rows.items(), key=lambda kv: -sum(kv[1]))
    for (name, grid), d in order[:top]:
        a = alone.get((name, grid), [])
        a_avg = f"{sum(a) / len(a) / 1e3:.2f}" if a else "-"
        print(f"| `{name}` | {grid} | {len(d)} | {sum(d) / len(d) / 1e3:.2f} | {min(d) / 1e3:.2f} | "
              f"{max(d) / 1e3:.2f} | {100.0 * sum(d) / total:.1f} | {len(a)} | {a_avg} |")
    print(f"\n{sum(len(v) for v in rows.values())} dispatches, {total / 1e6:.3f} ms of kernel time in total")


def counters(dirs, top, copy_mib):
    acc = collections.defaultdict(lambda: collections.defaultdict(list))
    dur = collections.defaultdict(list)
    for dirname in dirs:
        for path in find(dirname, "_counter_collection.csv"):
            with open(path, newline="") as f:
                for r in csv.DictReader(f):
                    key = (short_name(r["Kernel_Name"]), int(r["Grid_Size"]))
                    acc[key][r["Counter_Name"]].append(float(r["Counter_Value"]))
                    dur[key].append(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]))
    names = sorted({c for v in acc.values() for c in v})
    mean = lambda xs: sum(xs) / len(xs) if xs else float("nan")
    scale = {}
    copy_bytes = copy_mib * (1 << 20)
    copies = [k for k in acc if k[0].startswith("copy_kernel")]
    if copies:
        v = acc[max(copies, key=lambda k: k[1])]  # the yardstick is the largest copy of the run
        for c in ("FETCH_SIZE", "WRITE_SIZE"):
            if c in v:
                scale[c] = copy_bytes / (mean(v[c]) * 1024.0)
    if scale:
        print("counter scale from copy_kernel (%d MiB read, %d MiB written; counters in KiB): "
              % (copy_mib, copy_mib) + ", ".join(f"{c} x{s:.4f}" for c, s in sorted(scale.items())) + "\n")
    head = ["kernel", "grid", "dispatches"] + names + [c + " bytes (scaled)" for c in sorted(scale)]
    print("| " + " | ".join(head) + " |")
    print("|---|" + "---:|" * (len(head) - 1))
    order = sorted(acc.items(), key=lambda kv: -sum(dur[kv[0]]))
    for (name, grid), v in order[:top]:
        n = max(len(x) for x in v.values())
        cells = [f"`{name}`", str(grid), str(n)] + [f"{mean(v.get(c, [])):.4g}" for c in names]
        cells += [f"{mean(v.get(c, [])) * 1024.0 * scale[c]:.4g}" for c in sorted(scale)]
        print("| " + " | ".join(cells) + " |")


def read_dispatches(dirname):
    """[(order key, symbol, grid, duration ns, {counter: value})] of a trace directory, in dispatch order."""
    by_id = {}
    try:
        for path in find(dirname, "_counter_collection.csv"):
            with open(path, newline="") as f:
                for r in csv.DictReader(f):
                    key = (int(r["Dispatch_Id"]) if r.get("Dispatch_Id") else int(r["Start_Timestamp"]),)
                    d = by_id.setdefault(key, [short_name(r["Kernel_Name"]), int(r["Grid_Size"]),
                                               int(r["End_Timestamp"]) - int(r["Start_Timestamp"]), {}])
                    d[3][r["Counter_Name"]] = d[3].get(r["Counter_Name"], 0.0) + float(r["Counter_Value"])
    except SystemExit:
        pass
    if not by_id:
        for path in find(dirname, "_kernel_trace.csv"):
            with open(path, newline="") as f:
                for r in csv.DictReader(f):
                    grid = int(r["Grid_Size"]) if "Grid_Size" in r else \
                        int(r["Grid_Size_X"]) * int(r["Grid_Size_Y"]) * int(r["Grid_Size_Z"])
                    by_id[(int(r["Start_Timestamp"]),)] = [short_name(r["Kernel_Name"]), grid,
                                                          int(r["End_Timestamp"]) - int(r["Start_Timestamp"]), {}]
    return [(k, *v) for k, v in sorted(by_id.items())]


def marked_steps(disp, length):
    """The runs of `length` dispatches that stand between two marks (three fill kernel launches of
    one grid size in a row)."""
    is_fill = [d[1].startswith("fill_zero_kernel") for d in disp]
    marks = []  # index of the first dispatch behind a mark
    i = 0
    while i < len(disp):
        if is_fill[i]:
            j = i
            while j < len(disp) and is_fill[j] and disp[j][2] == disp[i][2]:
                j += 1
            if j - i == 3:
                marks.append((i, j))
            i = j
        else:
            i += 1
    return [disp[b:a2] for (_, b), (a2, _) in zip(marks, marks[1:]) if a2 - b == length]


def tags(dirs, sequence_file, merge, copy_mib):
    import json
    with open(sequence_file) as f:
        seq = json.load(f)
    workload, sequence = seq["workload"], seq["sequence"]
    per_tag = collections.OrderedDict((t, {"kernel": None, "grid": None, "ns": [], "counters": collections.defaultdict(list)})
                                      for t in sequence)
    scale = {}
    for dirname in dirs:
        disp = read_dispatches(dirname)
        steps = marked_steps(disp, len(sequence))
        if not steps:
            raise SystemExit(f"{dirname}: no marked step of {len(sequence)} dispatches found")
        for step in steps:
            if [d[1] for d in step] != [d[1] for d in steps[0]]:
                raise SystemExit(f"{dirname}: the marked steps launch different kernels: the trace is not of this run")
            for tag, (_, sym, grid, ns, ctr) in zip(sequence, step):
                rec = per_tag[tag]
                if rec["kernel"] is None:
                    rec["kernel"], rec["grid"] = sym, grid
                elif sym not in rec["kernel"].split(" + "):  # a tag may cover launches of several kernels
                    rec["kernel"] += " + " + sym
                if not ctr:
                    rec["ns"].append(ns)
                for c, v in ctr.items():
                    rec["counters"][c].append(v)
        copies = [d for d in disp if d[1].startswith("copy_kernel")]
        if copies:  # the yardstick is the largest copy of the run
            big = max(d[2] for d in copies)
            for c in ("FETCH_SIZE", "WRITE_SIZE"):
                v = [d[4][c] for d in copies if d[2] == big and c in d[4]]
                if v:
                    scale[c] = copy_mib * (1 << 20) / (sum(v) / len(v) * 1024.0)
    mean = lambda xs: sum(xs) / len(xs) if xs else float("nan")
    names = sorted({c for r in per_tag.values() for c in r["counters"]})
    if scale:
        print("counter scale from copy_kernel (%d MiB read, %d MiB written; counters in KiB): "
              % (copy_mib, copy_mib) + ", ".join(f"{c} x{s:.4f}" for c, s in sorted(scale.items())) + "\n")
    head = ["tag", "kernel", "grid", "launches per step", "avg us"] + names + [c + " bytes (scaled)" for c in sorted(scale)]
    print("| " + " | ".join(head) + " |")
    print("|---|---|" + "---:|" * (len(head) - 2))
    out = {}
    for tag, r in per_tag.items():
        cells = [f"`{tag}`", f"`{r['kernel']}`", str(r["grid"]), str(sequence.count(tag)),
                 f"{mean(r['ns']) / 1e3:.2f}" if r["ns"] else "-"]
        cells += [f"{mean(r['counters'].get(c, [])):.4g}" for c in names]
        cells += [f"{mean(r['counters'].get(c, [])) * 1024.0 * scale[c]:.4g}" for c in sorted(scale)]
        print("| " + " | ".join(cells) + " |")
        if "FETCH_SIZE" in scale and "WRITE_SIZE" in scale:
            fb = mean(r["counters"]["FETCH_SIZE"]) * 1024.0 * scale["FETCH_SIZE"]
            wb = mean(r["counters"]["WRITE_SIZE"]) * 1024.0 * scale["WRITE_SIZE"]
            out[tag] = {"kernel": r["kernel"], "grid": r["grid"], "fetch_bytes": round(fb), "write_bytes": round(wb),
                        "hbm_bytes_per_launch": round(fb + wb)}
    if merge and out:
        try:
            with open(merge) as f:
                js = json.load(f)
        except OSError:
            js = {}
        js.setdefault("workloads", {})[workload] = out
        js["scale"] = {c: round(v, 4) for c, v in scale.items()}
        with open(merge, "w") as f:
            json.dump(js, f, indent=1)
        print(f"\n{len(out)} tags of {workload} written to {merge}")


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("mode", choices=("kernels", "counters", "tags"))
    ap.add_argument("--sequence", help="tags: the file bench.py --sequence-out wrote in the traced run")
    ap.add_argument("--merge", help="tags: JSON file that takes the scaled bytes per launch")
    ap.add_argument("dirs", nargs="+")
    ap.add_argument("--top", type=int, default=40)
    ap.add_argument("--copy-mib", type=int, default=256)
    a = ap.parse_args()
    if a.mode == "tags":
        if not a.sequence:
            raise SystemExit("tags needs --sequence")
        tags(a.dirs, a.sequence, a.merge, a.copy_mib)
    elif a.mode == "kernels":
        kernels(a.dirs[0], a.top)
    else:
        counters(a.dirs, a.top, a.copy_mib)


if __name__ == "__main__":
    sys.exit(main())
