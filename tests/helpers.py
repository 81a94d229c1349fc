"""Shared synthetic-input builders for the tests (seeded, numpy on the host)."""
from __future__ import annotations

import numpy as np

from oracle import cards as ocards

H = 1326


def C(r: int, s: int) -> int:
    return s * 13 + r


def parse_board(text: str) -> list[int]:
    ranks = "23456789TJQKA"
    suits = "shdc"  # suit letters only need to be consistent inside one test
    return [suits.index(t[1]) * 13 + ranks.index(t[0]) for t in text.split()]


def random_boards(rng: np.random.Generator, m: int, k: int = 5) -> np.ndarray:
    return np.stack([rng.permutation(52)[:k] for _ in range(m)]).astype(np.int64)


def random_ranges(rng: np.random.Generator, boards: np.ndarray, alpha: float = 0.5) -> np.ndarray:
    """[M,2,1326] float32: Gamma(alpha) draws, board-blocked combos zeroed, rows normalised
    (a Dirichlet(alpha) sample over the allowed combos)."""
    allowed, _ = ocards.allowed_hands_for_boards(boards)
    x = rng.gamma(alpha, size=(boards.shape[0], 2, H)).astype(np.float32)
    x *= allowed[:, None, :]
    x /= x.sum(axis=-1, keepdims=True)
    return x.astype(np.float32)


def random_tree(rng: np.random.Generator, n_roots: int, depth: int, max_children: int = 5):
    """A random sparse tree in the evaluator's layout (level-major, children of one parent
    contiguous).  Returns a dict of int64 arrays."""
    offsets = [0, n_roots]
    parent = [-1] * n_roots
    child_count = []
    for d in range(depth):
        start, end = offsets[-2], offsets[-1]
        level = []
        for p in range(start, end):
            k = int(rng.integers(0, max_children + 1)) if d > 0 else int(rng.integers(1, max_children + 1))
            child_count.append(k)
            level += [p] * k
        if not level:
            break
        parent += level
        offsets.append(len(parent))
    total = len(parent)
    child_count += [0] * (total - len(child_count))
    child_count = np.asarray(child_count, dtype=np.int64)
    child_offsets = offsets[1] + np.cumsum(child_count) - child_count
    to_act = rng.integers(0, 2, size=total).astype(np.int64)
    parent = np.asarray(parent, dtype=np.int64)
    prev_actor = np.full(total, -1, dtype=np.int64)
    prev_actor[n_roots:] = to_act[parent[n_roots:]]
    root_index = np.arange(total)
    for i in range(n_roots, total):
        root_index[i] = root_index[parent[i]]
    top = offsets[-2] if len(offsets) > 2 else n_roots
    return dict(depth_offsets=offsets, parent_index=parent, child_count=child_count, child_offsets=child_offsets,
                to_act=to_act, prev_actor=prev_actor, root_index=root_index.astype(np.int64), total=total,
                top=top, bottom=n_roots)


def tree_as_dict(t):
    """The arrays of a SparseTree that oracle.cfr.OracleCFR takes."""
    d = {k: getattr(t, k) for k in ("depth_offsets", "parent_index", "action_from_parent", "child_count",
                                    "child_offsets", "prev_actor", "legal_mask", "leaf_mask", "new_street_mask",
                                    "fold_mask", "showdown_mask", "reward")}
    d.update({k: t.state[k] for k in ("to_act", "done", "scale")})
    d["showdown_potential"] = t.showdown_potential
    return d
