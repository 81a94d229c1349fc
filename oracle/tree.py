"""Betting rules and sparse-tree expansion, scalar restatement (one Python
object per node).  TEST INFRASTRUCTURE ONLY.

Follows ``src/p2/env/hunl_tensor_env.py``:
  legal_bins        <- legal_bins_amounts_and_mask   :348-423
  step              <- step_bins / step              :728-992 (betting part)
                       bet :684-705, finish_and_assign_rewards :707-724
and ``src/p2/search/sparse_cfr_evaluator.py``:
  build_tree        <- _construct_subgame            :142-306 (expansion loop
                       :167-197, node classes :227-260, fold values :296-300,
                       showdown potential :245-253)

All chip quantities are integers; a pot-fraction bet is
``trunc(float32(fraction) * float32(pot))`` (float32 product, as the reference
multiplies a float32 bin tensor by the pot).  River showdowns are marked
``done`` with ``street == 4``; who wins there depends on private cards and is
not part of the public tree.

Pinned by ``tests/golden/tree_golden.npz`` (written by running the reference
env itself over river / turn / flop roots, several bin sets and depths) and by
the hand-derived 21-node river tree (root 4 children, then 4, 5, 5, 2).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field

import numpy as np


@dataclass
class Node:
    to_act: int
    button: int
    street: int
    pot: int
    stacks: list
    committed: list
    min_raise: int
    actions_this_round: int
    is_allin: list
    starting_stacks: list
    scale: float
    done: bool = False
    reward: float = 0.0
    parent: int = -1
    action: int = -1
    children: list = field(default_factory=list)


def legal_bins(n: Node, bins: list[float]) -> tuple[list[int], list[bool]]:
    nb = len(bins) + 3
    amounts = [-1] * nb
    mask = [False] * nb
    me, opp = n.to_act, 1 - n.to_act
    to_call = n.committed[opp] - n.committed[me]
    mask[0] = to_call > 0
    mask[1] = True
    can_raise = n.stacks[me] > 0 and n.stacks[opp] > 0
    for i, frac in enumerate(bins):
        additional = int(np.float32(frac) * np.float32(n.pot))  # trunc toward 0
        amount = to_call + additional
        amounts[2 + i] = amount
        mask[2 + i] = can_raise and amount <= n.stacks[me] and additional >= n.min_raise
    amounts[nb - 1] = n.stacks[me]
    mask[nb - 1] = n.stacks[me] > 0
    if n.is_allin[opp]:
        mask[0] = mask[1] = True
        for i in range(2, nb):
            mask[i] = False
    if n.is_allin[me]:
        mask = [False] * nb
        mask[1] = True
    if n.done:
        mask = [False] * nb
    return amounts, mask


def step(parent: Node, bin_index: int, bins: list[float], bb: int) -> Node:
    n = copy.deepcopy(parent)
    n.children = []
    nb = len(bins) + 3
    amounts, _ = legal_bins(parent, bins)
    me, opp = n.to_act, 1 - n.to_act
    to_call = n.committed[opp] - n.committed[me]

    def pay(chips: int) -> None:
        n.stacks[me] -= chips
        n.committed[me] += chips
        n.pot += chips

    if bin_index == 0:
        n.done = True
        winner = opp
        pot = np.float32(n.pot)
        share = pot if winner == 0 else np.float32(0.0)
        n.reward = float(
            (np.float32(n.stacks[0]) + share - np.float32(n.starting_stacks[0]))
            / np.float32(n.scale)
        )
    elif bin_index == 1:
        pay(min(to_call, n.stacks[me]))
    elif bin_index == nb - 1:
        pay(n.stacks[me])
        n.is_allin[me] = True
    else:
        amt = amounts[bin_index]
        pay(amt)
        n.min_raise = max(n.min_raise, amt - to_call)
    n.to_act = 1 - n.to_act
    n.actions_this_round += 1

    equal = n.committed[0] == n.committed[1]
    allin_closed = (
        (n.is_allin[0] and n.is_allin[1])
        or (n.is_allin[0] and n.committed[0] <= n.committed[1])
        or (n.is_allin[1] and n.committed[1] <= n.committed[0])
    )
    if (not n.done) and (equal or allin_closed) and n.actions_this_round >= 2:
        n.committed = [0, 0]
        n.actions_this_round = 0
        n.to_act = 1 - n.button
        n.min_raise = bb
        if n.street == 3:
            n.done = True  # showdown
        n.street += 1
    return n


def build_tree(roots: list[Node], bins: list[float], depth: int, bb: int = 100) -> dict:
    """Breadth-first expansion to ``depth`` plies; nodes whose betting round has
    just closed (``actions_this_round == 0``) are not expanded below the root
    level.  Returns numpy arrays in the evaluator's row order (level-major,
    parent-major, action-ascending)."""
    nodes: list[Node] = [copy.deepcopy(r) for r in roots]
    offsets = [0, len(nodes)]
    d = 0
    while d < depth:
        start, end = offsets[-2], offsets[-1]
        new_nodes = []
        for p in range(start, end):
            par = nodes[p]
            _, mask = legal_bins(par, bins)
            if d > 0 and par.actions_this_round == 0:
                continue
            for a, ok in enumerate(mask):
                if ok:
                    c = step(par, a, bins, bb)
                    c.parent = p
                    c.action = a
                    new_nodes.append(c)
        if not new_nodes:
            break
        nodes.extend(new_nodes)
        offsets.append(len(nodes))
        d += 1

    total = len(nodes)
    n_roots = len(roots)
    nb = len(bins) + 3
    arr = lambda f, dt: np.asarray([f(x) for x in nodes], dtype=dt)  # noqa: E731
    out = {
        "depth_offsets": list(offsets),
        "parent_index": arr(lambda x: x.parent, np.int64),
        "action_from_parent": arr(lambda x: x.action, np.int64),
        "to_act": arr(lambda x: x.to_act, np.int64),
        "street": arr(lambda x: x.street, np.int64),
        "pot": arr(lambda x: x.pot, np.int64),
        "min_raise": arr(lambda x: x.min_raise, np.int64),
        "actions_this_round": arr(lambda x: x.actions_this_round, np.int64),
        "done": arr(lambda x: x.done, bool),
        "stacks": arr(lambda x: x.stacks, np.int64),
        "committed": arr(lambda x: x.committed, np.int64),
        "is_allin": arr(lambda x: x.is_allin, bool),
        "starting_stacks": arr(lambda x: x.starting_stacks, np.int64),
        "scale": arr(lambda x: x.scale, np.float32),
        "reward": arr(lambda x: x.reward, np.float32),
        "button": arr(lambda x: x.button, np.int64),
    }
    legal = np.zeros((total, nb), dtype=bool)
    for i, x in enumerate(nodes):
        legal[i] = legal_bins(x, bins)[1]
    out["legal_mask"] = legal
    is_root = np.zeros(total, dtype=bool)
    is_root[:n_roots] = True
    new_street = (out["actions_this_round"] == 0) & ~is_root
    leaf = out["done"] | new_street
    leaf[offsets[-2]:] = True
    child_mask = legal & ~leaf[:, None]
    child_count = child_mask.sum(axis=1).astype(np.int64)
    assert total == n_roots + int(child_count.sum())
    out["new_street_mask"] = new_street
    out["leaf_mask"] = leaf
    out["child_count"] = child_count
    out["child_offsets"] = offsets[1] + np.cumsum(child_count) - child_count
    prev_actor = np.full(total, -1, dtype=np.int64)
    prev_actor[n_roots:] = out["to_act"][out["parent_index"][n_roots:]]
    out["prev_actor"] = prev_actor
    out["fold_mask"] = (out["action_from_parent"] == 0) & out["done"]
    out["showdown_mask"] = out["street"] == 4
    out["showdown_potential"] = out["stacks"] + out["pot"][:, None] - out["starting_stacks"]
    return out


def make_preflop_root(starting0: int, starting1: int, button: int = 0, sb: int = 50, bb: int = 100) -> Node:
    """The state the env's reset leaves (``hunl_tensor_env.py:293-317``): the button has posted
    the small blind and acts first, the other player the big blind."""
    committed = [sb if p == button else bb for p in range(2)]
    return Node(to_act=button, button=button, street=0, pot=sb + bb,
                stacks=[starting0 - committed[0], starting1 - committed[1]], committed=committed, min_raise=bb,
                actions_this_round=0, is_allin=[False, False], starting_stacks=[starting0, starting1],
                scale=float(starting0))


def make_root(street: int, pot: int, stack0: int, stack1: int, button: int = 0,
              bb: int = 100, starting: tuple[int, int] | None = None,
              scale: float | None = None) -> Node:
    """A root at the start of a betting round: nothing committed, first to act
    is the non-button player (``hunl_tensor_env.py:892``).  By default each
    player is taken to have put half the pot in already."""
    if starting is None:
        starting = (stack0 + pot // 2, stack1 + pot // 2)
    if scale is None:
        scale = float(starting[0])
    return Node(to_act=1 - button, button=button, street=street, pot=pot,
                stacks=[stack0, stack1], committed=[0, 0], min_raise=bb,
                actions_this_round=0, is_allin=[False, False],
                starting_stacks=list(starting), scale=scale)
