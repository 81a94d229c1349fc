"""CPU: the product's vectorised tree builder and the oracle's scalar one against the
fixture written by the reference's own HUNLTensorEnv, and against each other."""
import os

import numpy as np
import pytest

from oracle import tree as OT
from poker2_amd.tree import RootStates, build_sparse_tree

STATE_KEYS = ["to_act", "street", "pot", "min_raise", "actions_this_round", "done", "stacks", "committed",
              "is_allin", "starting_stacks", "scale"]


def cases(golden_dir):
    g = np.load(os.path.join(golden_dir, "tree_golden.npz"))
    for name in sorted({k.split("/")[0] for k in g.files}):
        yield name, {k.split("/")[1]: g[k] for k in g.files if k.startswith(name + "/")}


def roots_of(case):
    r = case["roots"]
    pot, stacks, button = r[:, 0], r[:, 1:3], r[:, 3]
    street = int(case["root_street"])
    sb, bb = (int(x) for x in case["blinds"]) if "blinds" in case else (50, 100)
    if street == 0:      # reset state: the row holds the starting stacks
        return (RootStates.preflop(len(r), starting_stacks=stacks, button=button, sb=sb, bb=bb),
                [OT.make_preflop_root(int(s[0]), int(s[1]), button=int(b), sb=sb, bb=bb) for s, b in zip(stacks, button)],
                bb)
    prod = RootStates.at_round_start(street, pot, stacks, np.full((len(r), 5), -1), button=button, bb=bb)
    orac = [OT.make_root(street, int(p), int(s[0]), int(s[1]), button=int(b), bb=bb) for p, s, b in zip(pot, stacks, button)]
    return prod, orac, bb


def test_builders_match_reference_env_fixture(golden_dir):
    n = 0
    for name, case in cases(golden_dir):
        bins = [float(x) for x in case["bins"]]
        depth = int(case["depth"])
        prod, orac, bb = roots_of(case)
        t = build_sparse_tree(prod, bins, depth)
        o = OT.build_tree(orac, bins, depth, bb=bb)
        assert t.depth_offsets == list(case["depth_offsets"]) == o["depth_offsets"], name
        assert np.array_equal(t.parent_index, case["parent_index"]) and np.array_equal(o["parent_index"], case["parent_index"])
        assert np.array_equal(t.action_from_parent, case["action_from_parent"])
        assert np.array_equal(o["action_from_parent"], case["action_from_parent"])
        for k in STATE_KEYS:
            assert np.array_equal(t.state[k], case[k].astype(t.state[k].dtype)), (name, k)
            assert np.array_equal(o[k], case[k].astype(o[k].dtype)), (name, k)
        assert np.array_equal(t.legal_mask, case["legal_mask"]) and np.array_equal(o["legal_mask"], case["legal_mask"])
        fm = t.fold_mask
        assert np.array_equal(fm, o["fold_mask"])
        assert np.array_equal(t.reward[fm], case["reward"][fm]) and np.array_equal(o["reward"][fm], case["reward"][fm])
        for k in ("child_count", "child_offsets", "prev_actor", "leaf_mask", "new_street_mask", "showdown_mask"):
            assert np.array_equal(getattr(t, k), o[k]), (name, k)
        assert np.array_equal(t.showdown_potential, o["showdown_potential"])
        n += 1
    assert n >= 9


def test_hand_derived_river_tree():
    # pot 200, stacks 800/800, bins {0.5, 1}: root 4 children, then 4, 5, 5, 2 -> 21 nodes
    roots = RootStates.at_round_start(3, [200], [[800, 800]], np.arange(5)[None])
    t = build_sparse_tree(roots, [0.5, 1.0], 2)
    assert t.depth_offsets == [0, 1, 5, 21]
    assert t.child_count[:5].tolist() == [4, 4, 5, 5, 2]
    assert t.action_from_parent[1:5].tolist() == [1, 2, 3, 4]
    assert t.root_index.tolist() == [0] * 21
    # check-check is a showdown worth half the pot to either player
    sd = np.nonzero(t.showdown_mask)[0]
    assert 5 in sd and t.showdown_potential[5].tolist() == [100, 100]
    # folding to the half-pot bet: player 0 (first to act when button = 0 ... to_act = 1) loses nothing more
    assert t.fold_mask.sum() == 3


def test_full_river_tree_is_terminal_and_max_raises_extension():
    roots = RootStates.at_round_start(3, [200], [[800, 800]], np.arange(5)[None])
    full = build_sparse_tree(roots, [0.5, 1.0], 16)
    assert full.state["done"][full.leaf_mask].all()  # every leaf is a fold or a showdown
    capped = build_sparse_tree(roots, [0.5, 1.0], 16, max_raises=3)
    assert capped.state["done"][capped.leaf_mask].all()
    assert capped.total < full.total
    with pytest.raises(AssertionError):
        build_sparse_tree(RootStates.at_round_start(3, np.zeros(0), np.zeros((0, 2)), np.zeros((0, 5))), [0.5], 2)


def test_roots_from_an_env_like_object_with_torch_tensors():
    """RootStates.from_env reads the attribute names of the reference's HUNLTensorEnv
    (hunl_tensor_env.py:130-135,296) from torch tensors and selects rows."""
    import types

    import torch
    from poker2_amd.tree import RootStates, build_sparse_tree
    n = 5
    base = RootStates.at_round_start(3, np.arange(n) * 50 + 100, np.tile([[900, 700]], (n, 1)),
                                     np.tile(np.arange(5), (n, 1)), button=np.arange(n) % 2, bb=10)
    env = types.SimpleNamespace(bb=10)
    for name in ("street", "to_act", "button", "pot", "stacks", "committed", "min_raise", "actions_this_round",
                 "is_allin", "starting_stacks", "scale", "done"):
        setattr(env, name, torch.from_numpy(np.asarray(getattr(base, name))))
    env.board_indices = torch.from_numpy(base.board)
    idx = torch.tensor([4, 1, 2])
    roots = RootStates.from_env(env, idx)
    ref = base.select(np.array([4, 1, 2]))
    for name in RootStates.__dataclass_fields__:
        a, b = getattr(roots, name), getattr(ref, name)
        assert np.array_equal(a, b) if isinstance(a, np.ndarray) else a == b, name
    t1, t2 = build_sparse_tree(roots, [0.5, 1.0], 2), build_sparse_tree(ref, [0.5, 1.0], 2)
    assert t1.total == t2.total and np.array_equal(t1.child_count, t2.child_count)


def test_roots_of_the_flop_showdown_variant_are_refused():
    import types
    env = types.SimpleNamespace(flop_showdown=True)
    with pytest.raises(NotImplementedError):
        RootStates.from_env(env, np.arange(1))


@pytest.mark.parametrize("seed", range(12))
def test_work_items_partition_the_tree(seed):
    """split_work_items on random trees and cut levels: every family and every showdown row belongs to
    exactly one item; an item's rows lie under its head (tier 0: under its root) and inside its tier's
    levels; a showdown row sits in the item that owns its parent's family; inside a tier the items come in
    row order except for a tail of stated length that comes largest first (the whole tier when it is
    shorter than that); the tiers' counts add up."""
    from poker2_amd.tree import split_work_items
    rng = np.random.default_rng(900 + seed)
    n = int(rng.integers(1, 6))
    street = int(rng.integers(1, 4))
    bins = sorted(rng.choice([0.25, 0.5, 1.0, 2.0], size=int(rng.integers(1, 4)), replace=False).tolist())
    roots = RootStates.at_round_start(street, rng.integers(40, 900, n), rng.integers(30, 2500, (n, 2)),
                                      np.full((n, 5), -1), button=rng.integers(0, 2, n), bb=int(rng.choice([10, 100])))
    tree = build_sparse_tree(roots, bins, int(rng.integers(2, 7)), max_raises=[None, 2, 3][seed % 3])
    offs = np.asarray(tree.depth_offsets)
    level = np.searchsorted(offs, np.arange(tree.total), side="right") - 1
    has_children = tree.child_count > 0
    for cut, mid in ((1, None), (2, None), (2, 1), (9, None), (9, 1), (9, 2), (3, (1, 2)), (9, (1, 3))):
        tail = [10 ** 6, 3, 0][(seed + cut) % 3]        # longer than any tier / a few items / none
        it = split_work_items(tree, n, cut, mid, sorted_tail=tail)
        if it is None:
            assert len(offs) - 1 < 3 or not has_children[offs[1]:].any()
            continue
        assert sum(it.tiers) == len(it.item_root) == len(it.item_top) == len(it.parent_offsets) - 1
        assert it.tiers[0] == n and (it.item_top[:n] == 1).all() and (it.item_top[n:] == 0).all()
        assert len(it.tiers) == 1 + len(it.cuts) and it.n_sub == sum(it.tiers[1:])
        assert np.array_equal(np.sort(it.parents), np.nonzero(has_children)[0])            # each family once
        assert np.array_equal(np.sort(it.showdown), np.nonzero(tree.showdown_mask)[0])     # each showdown row once
        owner = np.full(tree.total, -1)
        bounds = [0] + list(it.cuts) + [len(offs) - 1]
        first_item = np.concatenate([[0], np.cumsum(it.tiers)])
        for tier in range(len(it.tiers)):
            for w in range(first_item[tier], first_item[tier + 1]):
                rows = it.parents[it.parent_offsets[w]:it.parent_offsets[w + 1]]
                assert (np.diff(rows) > 0).all()                                           # ascending: top-down order
                assert ((level[rows] >= bounds[tier]) & (level[rows] < bounds[tier + 1])).all()
                assert (tree.root_index[rows] == it.item_root[w]).all()
                if tier > 0:                                                               # one head per item, at the cut
                    heads = rows[level[rows] == bounds[tier]]
                    assert len(heads) == 1
                    up = rows.copy()
                    while (level[up] > bounds[tier]).any():
                        deeper = level[up] > bounds[tier]
                        up[deeper] = tree.parent_index[up[deeper]]
                    assert (up == heads[0]).all()
                owner[rows] = w
            if tier > 0:                       # order of the items, by the rows from the head down to the next cut
                hi_level = min(bounds[tier + 1], len(offs) - 2)
                below = np.arange(offs[bounds[tier]], offs[hi_level + 1])
                top = below.copy()
                while (level[top] > bounds[tier]).any():
                    deeper = level[top] > bounds[tier]
                    top[deeper] = tree.parent_index[top[deeper]]
                head_of = [it.parents[it.parent_offsets[w]] for w in range(first_item[tier], first_item[tier + 1])]
                rows_under = [int((top == h).sum()) for h in head_of]
                k = max(0, len(head_of) - tail)                                            # items before the tail
                assert all(a < b for a, b in zip(head_of[:k], head_of[1:k]))                # in row order
                assert all(a >= b for a, b in zip(rows_under[k:], rows_under[k + 1:]))      # then largest first
                assert sorted(head_of[k:]) == sorted(head_of)[k:]                          # the tail holds the last heads
        for w in range(len(it.item_root)):
            sd = it.showdown[it.showdown_offsets[w]:it.showdown_offsets[w + 1]]
            assert (owner[tree.parent_index[sd]] == w).all()                               # with its parent's family


def test_launch_order_keeps_row_order_and_sorts_the_tail():
    from poker2_amd.tree import launch_order
    size = np.array([5, 1, 9, 3, 3, 7, 2, 8])
    assert launch_order(size, 0).tolist() == list(range(8))
    assert launch_order(size, 3).tolist() == [0, 1, 2, 3, 4, 7, 5, 6]                     # 7, 2, 8 -> 8, 7, 2
    assert launch_order(size, 100).tolist() == [2, 7, 5, 0, 3, 4, 6, 1]                   # all by size, ties in row order
    assert launch_order(np.zeros(0, dtype=np.int64)).tolist() == []
