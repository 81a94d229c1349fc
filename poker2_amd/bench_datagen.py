"""One data-generation step at large batch: mixed flop / turn / river public belief states at the
start of a betting round, searched to the end of the street with a value network at the leaves,
then turned into training batches.

    python -m poker2_amd.bench_datagen [--roots 16384] [--iterations 64] [--max-raises 3] [--json]

Roots: random boards of 3 / 4 / 5 cards, Dirichlet(0.3) ranges with board-blocked hands removed,
pot uniform in 1..200 big blinds, stacks 100 big blinds, bet bins {0.5, 1} pot.  Network: 2 x 1326
ranges + board one-hot -> 3 x 1536 ReLU -> 2 x 1326, random weights, run under bf16 autocast.
Times (wall clock around device synchronisation) are reported for tree construction + state
allocation, the search, and ``training_data``; a first untimed pass warms the allocator.
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
from .leaf_models import NetworkLeafModel, RangeBoardMLP
from .tree import CARDS_ON_STREET, RootStates


def make_roots(b: int, seed: int):
    rng = np.random.default_rng(seed)
    street = rng.integers(1, 4, b)
    runout = np.argsort(rng.random((b, 52)), axis=1)[:, :5].astype(np.int64)
    board = np.where(np.arange(5)[None, :] < CARDS_ON_STREET[street][:, None], runout, -1)
    roots = RootStates.at_round_start(street, rng.integers(1, 201, b) * 100, np.full((b, 2), 10000), board,
                                      button=rng.integers(0, 2, b))
    roots.runout = runout
    cm = hand_combos_tensor().numpy()
    on = np.zeros((b, 53), bool)
    on[np.arange(b)[:, None], np.where(board >= 0, board, 52)] = True
    allowed = ~(on[:, cm[:, 0]] | on[:, cm[:, 1]])
    bel = torch.from_numpy(rng.gamma(0.3, size=(b, 2, 1326)).astype(np.float32) * allowed[:, None, :])
    return roots, bel / bel.sum(-1, keepdim=True)


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--roots", type=int, default=16384)
    ap.add_argument("--iterations", type=int, default=64)
    ap.add_argument("--max-raises", type=int, default=3)
    ap.add_argument("--spread-state", action="store_true",
                    help="the evaluator's placement option: the state tensors dealt to two slabs in different thirds "
                         "of the card's memory (set-up takes longer)")
    ap.add_argument("--reuse-state", action="store_true",
                    help="the evaluator keeps its state slabs from step to step (a placement is then paid for once)")
    ap.add_argument("--split", choices=["auto", "on", "off"], default="auto",
                    help="cut every root's tree into work items (auto: the evaluator's rule)")
    ap.add_argument("--json", action="store_true")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("bench_datagen needs a GPU (the product path has no CPU fallback)")
    dev = torch.device("cuda")
    b = args.roots
    roots, bel = make_roots(b, 5)
    model = NetworkLeafModel(RangeBoardMLP().to(dev), dev, autocast_dtype=torch.bfloat16)
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)
    ev = HipSparseCFREvaluator(model, dev, river_dcfr_config(b, iterations=args.iterations, depth=64), generator=gen,
                               max_raises=args.max_raises, spread_state=args.spread_state,
                               reuse_state=args.reuse_state,
                               split_small_batches={"auto": None, "on": True, "off": False}[args.split])

    def step():
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev.initialize_subgame(roots, np.arange(b), bel)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        nxt = ev.evaluate_cfr()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        ev.chance_helper.autocast_dtype = torch.bfloat16
        batches = ev.training_data()
        torch.cuda.synchronize()
        t3 = time.perf_counter()
        return (t1 - t0, t2 - t1, t3 - t2), nxt, batches
    step()
    (setup, search, data), nxt, (vb, pvb, pb) = step()
    out = {"roots": b, "nodes": ev.total_nodes, "model_leaves": int(ev.model_indices.numel()),
           "showdown_leaves": int(ev.showdown_indices.numel()), "iterations": args.iterations,
           "state_placed": bool(ev.state_placement.get("placed")),
           "placement_probe_ns_per_row": ([ev.state_placement["probe_ns_per_row_inside_first_slab"]] +
                                          ev.state_placement["probe_ns_per_row_candidates"])
           if ev.state_placement.get("placed") else None, "setup_s": setup, "search_s": search, "training_data_s": data, "ms_per_iteration": search / args.iterations * 1e3,
           "subgame_iterations_per_s": b * args.iterations / search, "public_states_per_s": b / (setup + search + data),
           "value_samples": len(vb) + len(pvb), "policy_samples": len(pb), "next_roots": nxt.roots.n,
           "peak_GiB": torch.cuda.max_memory_allocated() / 2**30}
    if args.json:
        print(json.dumps(out))
    else:
        for k, v in out.items():
            if isinstance(v, list):
                v = " ".join(f"{x:.1f}" for x in v)
            print(f"{k:28s} {v:.4g}" if isinstance(v, float) else f"{k:28s} {v}")


if __name__ == "__main__":
    main()
