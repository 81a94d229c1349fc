"""Writes tests/golden/tree_golden.npz by driving the reference's own
``p2.env.hunl_tensor_env.HUNLTensorEnv`` (pure torch, CPU) in the build
container.  Run once, here only:  python tests/golden/gen_tree_golden.py

The env module imports nothing but torch and ``p2.env.rules``; the evaluator
that normally owns the expansion loop (``sparse_cfr_evaluator.py:167-197``) is
not importable here (hydra / omegaconf are absent), so this script repeats that
breadth-first loop itself on top of the env's public methods
(``legal_bins_mask``, ``repeat_interleave``, ``step_bins``).  What the fixture
pins is the env's betting arithmetic: legality, bet sizing, min-raise, round
closure, fold rewards.  The fixture holds inputs and outputs only.
"""
from __future__ import annotations

import os
import sys

import numpy as np

REF_SRC = "/root/reference/src"
HERE = os.path.dirname(os.path.abspath(__file__))

# (name, street, bet_bins, depth, rows of (pot, stack0, stack1, button))
CASES = [
    ("river_b2_d2", 3, [0.5, 1.0], 2, [(200, 800, 800, 0), (200, 800, 800, 1)]),
    ("river_b2_d4", 3, [0.5, 1.0], 4, [(200, 800, 800, 0), (1000, 500, 500, 1), (150, 2000, 1000, 0)]),
    ("river_b2_d12", 3, [0.5, 1.0], 12, [(200, 800, 800, 0), (300, 120, 700, 1)]),
    ("river_b3_d3", 3, [0.33, 0.75, 1.5], 3, [(200, 800, 800, 0), (777, 1333, 901, 1), (90, 45, 300, 0)]),
    ("turn_b2_d3", 2, [0.5, 1.0], 3, [(200, 800, 800, 0), (400, 300, 900, 1)]),
    ("flop_b1_d2", 1, [1.0], 2, [(200, 900, 900, 1)]),
    # street 0: the roots are the env's reset state (blinds posted); the row holds (pot, starting stacks, button)
    ("preflop_b2_d4", 0, [0.5, 1.0], 4, [(150, 1000, 1000, 0), (150, 1000, 1000, 1)]),
    # the reference's own table (conf/config_rebel_cfr.yaml:66-70,72: blinds 5 / 10, 100 big blinds deep, depth 5);
    # a last element gives (small blind, big blind), 50 / 100 where absent
    ("preflop_deep_d5", 0, [0.5, 1.0], 5, [(15, 1000, 1000, 0), (15, 1000, 1000, 1), (15, 1700, 300, 0)], (5, 10)),
    ("flop_deep_d5", 1, [0.5, 1.0], 5, [(20, 990, 990, 1), (60, 970, 970, 0), (400, 800, 800, 1)], (5, 10)),
]


def main() -> None:
    sys.path.insert(0, REF_SRC)
    import torch
    from p2.env.hunl_tensor_env import HUNLTensorEnv

    out = {}
    for name, street, bins, depth, rows, *rest in CASES:
        n = len(rows)
        sb, bb = rest[0] if rest else (50, 100)
        env = HUNLTensorEnv(num_envs=n, starting_stack=1000, sb=sb, bb=bb,
                            default_bet_bins=list(bins), device=torch.device("cpu"))
        deck = torch.arange(9).repeat(n, 1)
        env.reset(force_button=torch.tensor([r[3] for r in rows]), force_deck=deck)
        for _ in range(2 * street):
            env.step_bins(torch.ones(n, dtype=torch.long))
        assert (env.street == street).all() and (env.actions_this_round == 0).all()
        if street == 0 and any(r[1] != 1000 or r[2] != 1000 for r in rows):
            # unequal starting stacks at the reset state: what reset leaves, with other stacks behind the blinds
            start = torch.tensor([[r[1], r[2]] for r in rows])
            env.stacks[:] = start - env.committed
            env.starting_stacks[:] = start
            env.scale[:] = start[:, 0].float()
        if street > 0:
            pot = torch.tensor([r[0] for r in rows])
            stacks = torch.tensor([[r[1], r[2]] for r in rows])
            env.pot[:] = pot
            env.stacks[:] = stacks
            env.starting_stacks[:] = stacks + (pot // 2)[:, None]
            env.scale[:] = env.starting_stacks[:, 0].float()

        levels = [env]
        parent_levels = [torch.full((n,), -1, dtype=torch.long)]
        action_levels = [torch.full((n,), -1, dtype=torch.long)]
        reward_levels = [torch.zeros(n)]
        offsets = [0, n]
        d = 0
        while d < depth:
            p_start, p_end = offsets[-2], offsets[-1]
            pe = levels[-1]
            legal = pe.legal_bins_mask()
            if d > 0:
                legal &= (pe.actions_this_round != 0)[:, None]
            counts = legal.sum(dim=-1)
            acts = torch.where(legal)[1]
            if acts.numel() == 0:
                break
            ne = pe.repeat_interleave(counts, output_size=acts.numel())
            par = torch.arange(p_start, p_end).repeat_interleave(counts, output_size=acts.numel())
            rew, _, _ = ne.step_bins(acts)
            levels.append(ne)
            parent_levels.append(par)
            action_levels.append(acts)
            reward_levels.append(rew.float())
            d += 1
            offsets.append(offsets[-1] + ne.N)

        def cat(attr):
            return torch.cat([getattr(e, attr) for e in levels]).numpy()

        full = HUNLTensorEnv.from_proto(levels[-1], num_envs=offsets[-1])
        cur = 0
        for e in levels:
            full.copy_state_from(e, torch.arange(e.N), torch.arange(cur, cur + e.N))
            cur += e.N
        out[f"{name}/bins"] = np.asarray(bins, dtype=np.float64)
        out[f"{name}/blinds"] = np.asarray([sb, bb], dtype=np.int64)
        out[f"{name}/depth"] = np.asarray(depth)
        out[f"{name}/roots"] = np.asarray(rows, dtype=np.int64)
        out[f"{name}/root_street"] = np.asarray(street)
        out[f"{name}/depth_offsets"] = np.asarray(offsets, dtype=np.int64)
        out[f"{name}/parent_index"] = torch.cat(parent_levels).numpy()
        out[f"{name}/action_from_parent"] = torch.cat(action_levels).numpy().astype(np.int8)
        out[f"{name}/reward"] = torch.cat(reward_levels).numpy().astype(np.float32)
        out[f"{name}/legal_mask"] = full.legal_bins_mask().numpy()
        for attr in ("to_act", "street", "pot", "min_raise", "actions_this_round", "done",
                     "stacks", "committed", "is_allin", "starting_stacks", "scale", "button"):
            out[f"{name}/{attr}"] = cat(attr)
        print(name, "nodes", offsets)
    np.savez_compressed(os.path.join(HERE, "tree_golden.npz"), **out)


if __name__ == "__main__":
    main()
