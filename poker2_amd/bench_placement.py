"""A map of how the card's memory treats a kernel that reads and writes many rows at once, depending on where
its arrays lie: the measurement behind the evaluator's ``spread_state`` option.

    python -m poker2_amd.bench_placement [--arena-gib 200] [--step-gib 4] [--anchors 0,70,140] [--json]

One large allocation stands in for the card's physical memory (a process cannot see physical addresses, but a
single large allocation is laid out regularly enough to show the structure).  ``p2hip_placement_probe`` streams
12 rows of 1326 floats in and 8 out per node, its 20 arrays dealt alternately to two windows of the allocation;
one window stays at an anchor offset, the other moves through the allocation.  On an MI355X the time per row
falls into two levels, about 25 ns when both windows lie in the same third of the card's memory and about 21 ns
when they lie in different thirds, and the offsets that are "the same third" as an anchor change with the
anchor: the allocation divides into three classes of offsets.  No counterpart in the reference.
"""
from __future__ import annotations

import argparse
import ctypes
import json

import torch

from . import _lib

GIB = 1 << 30
WINDOW_BYTES = 10 * 12288 * 1326 * 4            # ten of the probe's arrays at their largest


def probe_ns_per_row(a: int, b: int) -> float:
    ms = ctypes.c_float()
    _lib.call("p2hip_placement_probe", a, b, WINDOW_BYTES, 3, ctypes.byref(ms), _lib.stream_ptr())
    return float(ms.value) * 1e6 / 12288


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--arena-gib", type=int, default=200)
    ap.add_argument("--step-gib", type=float, default=4.0)
    ap.add_argument("--anchors", default="0,70,140", help="offsets (GiB) of the window that stays")
    ap.add_argument("--json", action="store_true")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("bench_placement needs a GPU")
    free, total = torch.cuda.mem_get_info()
    size = min(args.arena_gib * GIB, free - 8 * GIB)
    arena = torch.empty(size, dtype=torch.uint8, device="cuda")
    base, width = arena.data_ptr(), WINDOW_BYTES / GIB
    inside = probe_ns_per_row(base, base + WINDOW_BYTES)          # both windows side by side
    out = {"card_GiB": total / GIB, "arena_GiB": size / GIB, "window_GiB": width,
           "ns_per_row_two_windows_side_by_side": inside, "scans": []}
    for anchor in (float(x) for x in args.anchors.split(",")):
        if (anchor + width) * GIB > size:
            continue
        rows, d = [], 0.0
        while (d + width) * GIB <= size:
            if abs(d - anchor) >= width:
                ns = probe_ns_per_row(base + int(anchor * GIB) // 256 * 256, base + int(d * GIB) // 256 * 256)
                rows.append((d, ns))
            d += args.step_gib
        out["scans"].append({"anchor_GiB": anchor, "offset_GiB_and_ns_per_row": rows})
    if args.json:
        print(json.dumps(out))
        return
    print(f"card {out['card_GiB']:.1f} GiB, one allocation of {out['arena_GiB']:.0f} GiB, windows of {width:.2f} GiB; "
          f"two windows side by side: {inside:.1f} ns per row")
    for scan in out["scans"]:
        rows = scan["offset_GiB_and_ns_per_row"]
        lo = min(ns for _, ns in rows)
        same = [d for d, ns in rows if ns > 1.1 * lo]
        print(f"anchor at {scan['anchor_GiB']:.0f} GiB: " + " ".join(f"{d:.0f}:{ns:.1f}" for d, ns in rows))
        print(f"  offsets in the anchor's class (more than 1.1 x the fastest, {lo:.1f} ns): "
              + (" ".join(f"{d:.0f}" for d in same) if same else "none"))


if __name__ == "__main__":
    main()
