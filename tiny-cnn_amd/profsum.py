#!/usr/bin/env python3
"""Condenses rocprofv3 CSV output into the short tables kept under profiles/.

    python -m tiny-cnn_amd.profsum kernels  <dir>            # --kernel-trace --stats run
    python -m tiny-cnn_amd.profsum counters <dir> [<dir>..]  # --pmc runs (one counter set per dir)

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


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("mode", choices=("kernels", "counters"))
    ap.add_argument("dirs", nargs="+")
    ap.add_argument("--top", type=int, default=40)
    ap.add_argument("--copy-mib", type=int, default=256)
    a = ap.parse_args()
    if a.mode == "kernels":
        kernels(a.dirs[0], a.top)
    else:
        counters(a.dirs, a.top, a.copy_mib)


if __name__ == "__main__":
    sys.exit(main())
