"""Whole river searches, wall clock: tree construction + state set-up, the DCFR iterations with
their leaf sampling (``evaluate_cfr``), and the local exploitability afterwards.

    python -m poker2_amd.bench_search [--roots 1024] [--max-raises 3] [--depth 16] [--iterations 200] [--spread-state] [--json]

Roots: random 5-card boards, Gamma(0.5) ranges with board-blocked hands removed, pot 200, stacks
800 each, bet bins {0.5, 1.5} pot, no leaf network (river trees end in folds and showdowns).  The
reference's counterpart is ``CFREvaluator.evaluate_cfr`` (src/p2/search/cfr_evaluator.py:1497-1532)
after ``initialize_subgame`` (src/p2/search/cfr_evaluator.py:770) on the tree of
``SparseCFREvaluator._construct_subgame`` (src/p2/search/sparse_cfr_evaluator.py:142-306).  The first pass
warms the allocator and is not reported.
"""
from __future__ import annotations

import argparse
import json
import time

import numpy as np
import torch

from .card_utils import hand_combos_tensor
from .config import river_dcfr_config
from .evaluator import HipSparseCFREvaluator
from .tree import RootStates


def make_roots(n: int, seed: int):
    rng = np.random.default_rng(seed)
    boards = np.argsort(rng.random((n, 52)), axis=1)[:, :5].astype(np.int64)
    cm = hand_combos_tensor().numpy()
    on = np.zeros((n, 52), dtype=bool)
    on[np.arange(n)[:, None], boards] = True
    allowed = ~(on[:, cm[:, 0]] | on[:, cm[:, 1]])
    bel = rng.gamma(0.5, size=(n, 2, 1326)).astype(np.float32) * allowed[:, None, :]
    bel /= bel.sum(-1, keepdims=True)
    roots = RootStates.at_round_start(3, np.full(n, 200), np.tile([[800, 800]], (n, 1)), boards,
                                      button=np.arange(n) % 2)
    return roots, torch.from_numpy(bel)


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--roots", type=int, default=1024)
    ap.add_argument("--max-raises", type=int, default=3)
    ap.add_argument("--depth", type=int, default=16)
    ap.add_argument("--iterations", type=int, default=200)
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--spread-state", action="store_true",
                    help="the evaluator's placement option for long searches: faster iterations from 2048 roots on, "
                         "set-up seconds longer once the card's memory has been used before")
    ap.add_argument("--json", action="store_true")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("bench_search needs a GPU (the product path has no CPU fallback)")
    dev = torch.device("cuda")
    n = args.roots
    roots, bel = make_roots(n, args.seed)
    for _ in range(2):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        cfg = river_dcfr_config(n, iterations=args.iterations, depth=args.depth, dcfr_delay=0)
        ev = HipSparseCFREvaluator(None, dev, cfg, fused_iteration=True, max_raises=args.max_raises,
                                   spread_state=args.spread_state)
        ev.initialize_subgame(roots, np.arange(n), bel)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        ev.evaluate_cfr(training_mode=True)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        stats = ev._compute_exploitability()
        torch.cuda.synchronize()
        t3 = time.perf_counter()
    out = {"roots": n, "nodes": int(ev.total_nodes), "iterations": args.iterations,
           "spread_state": bool(args.spread_state), "state_placed": bool(ev.state_placement.get("placed")),
           "setup_s": t1 - t0, "search_s": t2 - t1, "exploitability_s": t3 - t2,
           "subgame_iterations_per_s": n * args.iterations / (t2 - t1),
           "local_exploitability": float(stats.local_exploitability.mean())}
    if args.json:
        print(json.dumps(out))
    else:
        placed = (" (state placed)" if out["state_placed"] else " (state not placed)") if args.spread_state else ""
        print(f"{n} roots, {out['nodes']} nodes: set-up {out['setup_s']:.3f} s{placed}, {args.iterations} iterations "
              f"{out['search_s']:.3f} s -> {out['subgame_iterations_per_s'] / 1e6:.3f} M subgame-iterations/s, "
              f"exploitability pass {1e3 * out['exploitability_s']:.1f} ms "
              f"(mean local exploitability {out['local_exploitability']:.4g})")


if __name__ == "__main__":
    main()
