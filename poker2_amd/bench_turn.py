"""Turn subgames whose leaves are chance nodes: every street-end leaf is expanded over the river cards
not on its board (blocked hands removed, ranges renormalised), a value network answers for the
samples, and the answers are averaged per leaf.

    python -m poker2_amd.bench_turn [--roots 512] [--max-raises 3] [--iterations 100] [--json]

Roots: random 4-card boards, Gamma(0.5) ranges with board-blocked hands removed, pot 200, stacks 800
each, bet bins {0.5, 1} pot.  Network: 2 x 1326 ranges + board one-hot -> 3 x 1536 ReLU -> 2 x 1326,
random weights, fp32.  The reference's counterpart is ``evaluate_cfr`` with
``ChanceNodeHelper.single_card_chance_values`` at the leaves (src/p2/search/chance_node_helper.py:360-479).
Reported: tree construction + state set-up, the DCFR iterations (wall clock around device
synchronisation), and the share of an iteration that the leaves take (expansion, network, mean).
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
from .leaf_models import ChanceLeafModel, RangeBoardMLP
from .tree import RootStates


def make_roots(b: int, seed: int):
    rng = np.random.default_rng(seed)
    boards = np.full((b, 5), -1, dtype=np.int64)
    boards[:, :4] = np.argsort(rng.random((b, 52)), axis=1)[:, :4]
    cm = hand_combos_tensor().numpy()
    on = np.zeros((b, 52), dtype=bool)
    on[np.arange(b)[:, None], boards[:, :4]] = True
    allowed = ~(on[:, cm[:, 0]] | on[:, cm[:, 1]])
    bel = rng.gamma(0.5, size=(b, 2, 1326)).astype(np.float32) * allowed[:, None, :]
    bel /= bel.sum(-1, keepdims=True)
    roots = RootStates.at_round_start(2, np.full(b, 200), np.tile([[800, 800]], (b, 1)), boards,
                                      button=np.arange(b) % 2)
    return roots, torch.from_numpy(bel)


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--roots", type=int, default=512)
    ap.add_argument("--max-raises", type=int, default=3)
    ap.add_argument("--iterations", type=int, default=100)
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--json", action="store_true")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("bench_turn needs a GPU (the product path has no CPU fallback)")
    dev = torch.device("cuda")
    b = args.roots
    roots, bel = make_roots(b, args.seed)
    torch.manual_seed(args.seed)
    model = ChanceLeafModel(RangeBoardMLP().to(dev), dev)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    cfg = river_dcfr_config(b, iterations=args.iterations, depth=16, dcfr_delay=0)
    ev = HipSparseCFREvaluator(model, dev, cfg, fused_iteration=True, max_raises=args.max_raises)
    ev.initialize_subgame(roots, np.arange(b), bel)
    ev.prepare_search()
    lean = dict(lean=True, alternate_reach_avg=True)       # as evaluate_cfr runs every iteration but its last
    for t in range(2):                       # first iterations: allocator, GEMM heuristics
        ev.cfr_iteration(t, **lean)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    for t in range(2, args.iterations):
        ev.cfr_iteration(t, **(lean if t + 1 < args.iterations else {}))
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    reps = 5
    for _ in range(reps):
        model.leaf_values(ev.beliefs[ev.model_indices], ev.model_indices, ev)
    torch.cuda.synchronize()
    t3 = time.perf_counter()
    per_iter = (t2 - t1) / max(1, args.iterations - 2)
    leaves = int(ev.model_indices.numel())
    out = {"roots": b, "nodes": int(ev.total_nodes), "chance_leaves": leaves, "network_samples": leaves * 48,
           "iterations": args.iterations, "setup_and_first_two_s": t1 - t0, "ms_per_iteration": 1e3 * per_iter,
           "subgame_iterations_per_s": b / per_iter, "leaf_evaluation_ms": 1e3 * (t3 - t2) / reps,
           "peak_GiB": torch.cuda.max_memory_allocated() / 2 ** 30}
    if args.json:
        print(json.dumps(out))
    else:
        for k, v in out.items():
            print(f"{k:28s} {v:.4g}" if isinstance(v, float) else f"{k:28s} {v}")


if __name__ == "__main__":
    main()
