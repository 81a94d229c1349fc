"""Self-play data generation around the search, MI355X path.

Mirror of ``RebelDataGenerator`` (src/p2/search/rebel_data_generator.py:11-95): same constructor
arguments, ``generate_data(value_sample_count)`` and loop — search the current public belief
states, hand the three training batches to the buffers, continue from the sampled leaves, refill
with freshly dealt hands.  ``EnvProto`` stands for the template env the reference clones and
resets (src/p2/env/hunl_tensor_env.py:58-72, 196-346): blinds, stacks and the generator that
deals.  Public states travel as ``RootStates`` (numpy, a few dozen bytes per state); ranges stay
on the GPU.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np
import torch

from .card_utils import NUM_HANDS
from .rebel_batch import RebelBatch
from .tree import RootStates
from ._guards import require as _req


@dataclass
class PublicBeliefState:
    """Public states and the ranges of both players in them (cfr_evaluator.py:55-91)."""
    env: RootStates
    beliefs: torch.Tensor      # [batch, 2, 1326]

    def __post_init__(self) -> None:
        _req(self.beliefs.shape[0] == self.env.n, "self.beliefs.shape[0] == self.env.n")


class EnvProto:
    """Deals new hands the way the reference env's ``reset`` does: a random button, nine cards
    off a shuffled deck (four hole cards nobody looks at during the search, five board cards kept
    as the hand's runout), blinds posted, optionally random stacks around ``mean_stack``.  The
    draws are made on the generator's device in the reference's order (button, deck, stacks), so
    a CPU generator with the same seed deals the same hands as the reference env."""

    def __init__(self, mean_stack: int, sb: int = 50, bb: int = 100, randomize_stacks: bool = False,
                 rng: torch.Generator | None = None) -> None:
        self.mean_stack, self.sb, self.bb = int(mean_stack), int(sb), int(bb)
        self.randomize_stacks = bool(randomize_stacks)
        self.rng = rng if rng is not None else torch.Generator(device="cpu")

    def _sample_starting_stacks(self, n: int) -> np.ndarray:
        """hunl_tensor_env.py:196-217."""
        min_stack = math.ceil(0.1 * self.mean_stack)
        total = 2 * self.mean_stack
        if min_stack * 2 > total:
            raise ValueError("mean_stack too small to satisfy minimum stack constraint")
        if not self.randomize_stacks or n == 0:
            return np.full((n, 2), self.mean_stack, dtype=np.int64)
        low, high = min_stack, total - min_stack
        rand = torch.rand(n, generator=self.rng, device=self.rng.device)
        p0 = (low + torch.floor(rand * (high - low + 1))).long().cpu().numpy()
        return np.stack([p0, total - p0], axis=1)

    def reset(self, n: int) -> RootStates:
        gdev = self.rng.device
        button = torch.randint(0, 2, (n,), generator=self.rng, device=gdev).cpu().numpy()
        random_vals = torch.rand(n, 52, generator=self.rng, device=gdev)
        deck = torch.topk(random_vals, 9, dim=1).indices.cpu().numpy()     # positions in an ordered deck = card ids
        stacks = self._sample_starting_stacks(n)
        roots = RootStates.preflop(n, starting_stacks=stacks, button=button, sb=self.sb, bb=self.bb)
        roots.runout = deck[:, 4:9].astype(np.int64)
        self.last_deck = deck          # the nine cards per hand of the latest reset, hole cards first
        return roots


def _overwrite_rows(dst: RootStates, src: RootStates, count: int) -> None:
    """dst[:count] = src[:count] for every per-state array."""
    if src.runout is None:
        raise ValueError("states that continue a hand must carry their runout")
    if dst.last_board is None:
        dst.last_board = dst.previous_board()
    src_last = src.previous_board()
    for name in RootStates.__dataclass_fields__:
        a = getattr(dst, name)
        b = src_last if name == "last_board" else getattr(src, name)
        if isinstance(a, np.ndarray):
            a[:count] = b[:count]


class RebelDataGenerator:
    def __init__(self, env_proto: EnvProto, evaluator, value_buffer, policy_buffer) -> None:
        self.env_proto = env_proto
        self.evaluator = evaluator
        self.value_buffer = value_buffer
        self.policy_buffer = policy_buffer
        self.device = evaluator.device
        self.current_pbs = self._new_pbs(evaluator.root_nodes)
        self.last_extra = 0

    def _new_pbs(self, target_batch_size: int) -> PublicBeliefState:
        beliefs = torch.full((target_batch_size, self.evaluator.num_players, NUM_HANDS), 1.0 / NUM_HANDS,
                             device=self.device)
        return PublicBeliefState(env=self.env_proto.reset(target_batch_size), beliefs=beliefs)

    def _top_up(self) -> PublicBeliefState:
        """The states the next search starts from: the hands still being played first, freshly dealt
        ones behind them until the evaluator's batch is full (:42-50, :60-66)."""
        want = self.evaluator.root_nodes
        playing = self.current_pbs
        if playing is not None and playing.env.n >= want:
            return playing
        fresh = self._new_pbs(want)
        if playing is not None:
            kept = playing.env.n
            _overwrite_rows(fresh.env, playing.env, kept)
            fresh.beliefs[:kept] = playing.beliefs
        return fresh

    def search_pass(self) -> tuple[RebelBatch, RebelBatch, RebelBatch]:
        """One search over a full batch of public states.  Its three training batches — values at the
        roots, values of the states before the deal, policies — go to the buffers in the reference's
        order (policy, value, pre-deal value: :70-77); the sampled leaves become the states that are
        still being played."""
        start = self._top_up()
        ev = self.evaluator
        ev.initialize_subgame(start.env, np.arange(start.env.n), start.beliefs)
        self.current_pbs = ev.evaluate_cfr()
        value, pre_deal_value, policy = ev.training_data()
        for buffer, batch in ((self.policy_buffer, policy), (self.value_buffer, value),
                              (self.value_buffer, pre_deal_value)):
            buffer.add_batch(batch)
        return value, pre_deal_value, policy

    def generate_data(self, value_sample_count: int) -> tuple[RebelBatch | None, RebelBatch | None]:
        """Runs search passes until ``value_sample_count`` root value samples exist, counting what the
        previous call produced beyond its own request (:52-95).  Returns (value batch, policy batch)
        of this call — the same batches that went to the buffers — or None where no pass ran."""
        have = self.last_extra
        values: list[RebelBatch] = []
        policies: list[RebelBatch] = []
        while have < value_sample_count:
            value, pre_deal_value, policy = self.search_pass()
            values += [value, pre_deal_value]
            policies.append(policy)
            have += len(value)
        self.last_extra = have - value_sample_count
        return (RebelBatch.cat(values) if values else None), (RebelBatch.cat(policies) if policies else None)
