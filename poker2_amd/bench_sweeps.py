"""Where a workgroup of the iteration kernel spends its time: the sweeps' shares, from the tuning build.

    python -m poker2_amd.build --sweep-timers          (once, beside the library; needs no GPU)
    python -m poker2_amd.bench_sweeps [--roots 4096] [--max-raises 3] [--depth 16] [--iterations 10] [--one-workgroup-per-root] [--plain]

The tuning build of the library (``-DP2_ITER_PROFILE``) adds the ticks of the 100 MHz wall clock that
each workgroup spends inside each sweep of ``cfr_iteration_kernel`` into a table in device memory; this
program runs river DCFR iterations on it (roots as in ``poker2_amd.bench_search``) and prints, per sweep,
the mean time per root and iteration and its share.  Workgroups overlap on a compute unit (three are
resident), so the figures are residence times, not exclusive ones: they say which sweep a workgroup
lives in, and sum to the workgroups' total residence, about three times the kernel's duration.  The
timers cost a few per cent themselves.  The product never loads this build.
"""
from __future__ import annotations

import argparse
import ctypes
import os

import numpy as np
import torch

from . import _lib
from .build import SWEEP_TIMER_LIB_PATH

SLOTS = [  # (slot in the kernel's table, label, part of)
    (0, "sweep 1: regrets, discounting, regret matching", None),
    (4, "  of which: opponent beliefs of the parents -> card sums", 0),
    (1, "sweep 2: reach, beliefs, average policy (top-down)", None),
    (6, "  of which: the family's block reduction", 1),
    (2, "sweep 3: leaf values and backup (bottom-up)", None),
    (3, "  of which: showdown leaves", 2),
    (5, "  of which: actor beliefs x policy -> card sums", 2),
]


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--roots", type=int, default=4096)
    ap.add_argument("--max-raises", type=int, default=3)
    ap.add_argument("--depth", type=int, default=16)
    ap.add_argument("--iterations", type=int, default=10)
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--one-workgroup-per-root", action="store_true",
                    help="no work items: every root's tree walked by one workgroup")
    ap.add_argument("--plain", action="store_true",
                    help="iterations that store every row, reach_avg in place (cfr_iteration(t)); default: as a search "
                         "runs them (rows nothing reads left unwritten, reach_avg alternating between two buffers)")
    args = ap.parse_args()
    how = {} if args.plain else dict(lean=True, alternate_reach_avg=True)
    if not torch.cuda.is_available():
        raise SystemExit("bench_sweeps needs a GPU")
    if not os.path.exists(SWEEP_TIMER_LIB_PATH):
        raise SystemExit(f"{SWEEP_TIMER_LIB_PATH} is missing: python -m poker2_amd.build --sweep-timers")
    _lib.LIB_PATH = SWEEP_TIMER_LIB_PATH          # before anything loads the library
    from . import evaluator as E
    from .bench_search import make_roots
    from .config import river_dcfr_config
    if args.one_workgroup_per_root:
        E.SPLIT_ROOTS_BELOW, E.SPLIT_NODES_PER_ROOT = 0, 10 ** 9
    lib = _lib.load()
    read = lib.p2hip_iter_prof_read
    read.argtypes, read.restype = [ctypes.c_void_p, ctypes.c_int], ctypes.c_int
    n = args.roots
    roots, bel = make_roots(n, args.seed)
    cfg = river_dcfr_config(n, iterations=args.iterations + 5, depth=args.depth, dcfr_delay=0)
    ev = E.HipSparseCFREvaluator(None, torch.device("cuda"), cfg, fused_iteration=True, max_raises=args.max_raises)
    ev.initialize_subgame(roots, np.arange(n), bel)
    ev.prepare_search()
    table = np.zeros((8192, 8), dtype=np.int64)
    for t in range(5):
        ev.cfr_iteration(t, **how)
    torch.cuda.synchronize()
    _lib.check(read(table.ctypes.data, 1), "p2hip_iter_prof_read")
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for t in range(5, 5 + args.iterations):
        ev.cfr_iteration(t, **how)
    stop.record()
    torch.cuda.synchronize()
    _lib.check(read(table.ctypes.data, 1), "p2hip_iter_prof_read")
    ticks = table.sum(0).astype(np.float64)                      # over all workgroups
    us = ticks / 100.0 / (n * args.iterations)                   # per root and iteration
    total = us[0] + us[1] + us[2]
    items = "one workgroup per root" if ev._items is None else f"work items in tiers of {list(ev._items.tiers)}"
    print(f"{n} river roots, {int(ev.total_nodes)} nodes ({ev.total_nodes // n} per root), {items}; "
          f"{args.iterations} {'plain' if args.plain else 'search'} iterations, "
          f"{start.elapsed_time(stop) / args.iterations:.3f} ms each with the timers")
    print(f"{'':58s} {'us / root-iteration':>20s} {'share':>7s}")
    for slot, label, parent in SLOTS:
        print(f"{label:58s} {us[slot]:20.1f} {100 * us[slot] / total:6.1f}%")
    label = "all sweeps (residence of the root's workgroups)"
    print(f"{label:58s} {total:20.1f}")


if __name__ == "__main__":
    main()
