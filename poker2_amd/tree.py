"""Sparse betting-tree construction on the host (numpy, all roots at once).

Produces the tree layout every kernel consumes -- the one the reference builds in
``SparseCFREvaluator._construct_subgame`` (src/p2/search/sparse_cfr_evaluator.py:142-306)
by stepping its tensor env: rows are level-major, the children of one parent are
contiguous and ordered by action bin, and a child's row holds the quantities "for
the action that leads to it".

The betting rules are those of src/p2/env/hunl_tensor_env.py (legality :348-423,
bet / fold reward :684-724, step and round closure :766-897): integer chips, a
pot-fraction bet is ``trunc(float32(fraction) * float32(pot))`` on top of the call,
all-in always available, a betting round closes after two actions when the
commitments match (or an all-in is covered), the river closes into a showdown.

``max_raises`` is an extension for synthetic benchmark trees (the reference caps by
ply depth only): once that many bets/raises were made in the round, only fold and
call remain.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from types import SimpleNamespace

import numpy as np
from ._guards import require as _req

H = 1326


CARDS_ON_STREET = np.array([0, 3, 4, 5, 5])   # board cards visible on streets 0..3 and at showdown


@dataclass
class RootStates:
    """Public state of N subgame roots (numpy arrays of length N)."""
    street: np.ndarray
    to_act: np.ndarray
    button: np.ndarray
    pot: np.ndarray
    stacks: np.ndarray            # [N,2]
    committed: np.ndarray         # [N,2]
    min_raise: np.ndarray
    actions_this_round: np.ndarray
    is_allin: np.ndarray          # [N,2] bool
    starting_stacks: np.ndarray   # [N,2]
    scale: np.ndarray             # [N] float32
    board: np.ndarray             # [N,5] int64, -1 = not dealt
    done: np.ndarray = None       # [N] bool
    bb: int = 100
    last_board: np.ndarray = None  # [N,5] board before the latest action (None: derived, see previous_board)
    runout: np.ndarray = None      # [N,5] the complete board these roots will see (None: cards are drawn when needed)

    def __post_init__(self):
        if self.done is None:
            self.done = np.zeros(self.street.shape[0], dtype=bool)
        if self.runout is not None:
            shown = np.arange(5)[None, :] < CARDS_ON_STREET[np.clip(self.street, 0, 4)][:, None]
            _req(np.array_equal(np.where(shown, self.runout, -1), self.board), "runout does not continue the board")

    def previous_board(self) -> np.ndarray:
        """The env's ``last_board_indices`` (src/p2/env/hunl_tensor_env.py:862): every action saves the
        board before cards are dealt, so a root at the start of a betting round still holds the
        previous street's board and any other root its own."""
        if self.last_board is not None:
            return self.last_board
        street = np.clip(self.street, 0, 4)
        at_start = (self.actions_this_round == 0) & (street >= 1)
        keep = np.where(at_start, CARDS_ON_STREET[np.maximum(street - 1, 0)], 5)
        return np.where(np.arange(5)[None, :] < keep[:, None], self.board, -1)

    @property
    def n(self) -> int:
        return int(self.street.shape[0])

    def select(self, idx) -> "RootStates":
        """Rows ``idx`` as a new RootStates."""
        idx = np.asarray(idx)
        kw = {}
        for name in self.__dataclass_fields__:
            v = getattr(self, name)
            kw[name] = v[idx] if isinstance(v, np.ndarray) else v
        return RootStates(**kw)

    @classmethod
    def at_round_start(cls, street, pot, stacks, board, button=0, bb: int = 100,
                       starting_stacks=None, scale=None) -> "RootStates":
        """Roots at the start of a betting round: nothing committed, the non-button player
        acts first.  By default each player is taken to have paid half the pot already."""
        pot = np.atleast_1d(np.asarray(pot, dtype=np.int64))
        n = pot.shape[0]
        stacks = np.broadcast_to(np.asarray(stacks, dtype=np.int64), (n, 2)).copy()
        button = np.broadcast_to(np.asarray(button, dtype=np.int64), (n,)).copy()
        street = np.broadcast_to(np.asarray(street, dtype=np.int64), (n,)).copy()
        if starting_stacks is None:
            starting_stacks = stacks + (pot // 2)[:, None]
        starting_stacks = np.broadcast_to(np.asarray(starting_stacks, dtype=np.int64), (n, 2)).copy()
        if scale is None:
            scale = starting_stacks[:, 0].astype(np.float32)
        scale = np.broadcast_to(np.asarray(scale, dtype=np.float32), (n,)).copy()
        board = np.asarray(board, dtype=np.int64)
        if board.ndim == 1:
            board = np.broadcast_to(board, (n, board.shape[0]))
        full = np.full((n, 5), -1, dtype=np.int64)
        full[:, : board.shape[1]] = board
        return cls(street=street, to_act=1 - button, button=button, pot=pot, stacks=stacks,
                   committed=np.zeros((n, 2), np.int64), min_raise=np.full(n, bb, np.int64),
                   actions_this_round=np.zeros(n, np.int64), is_allin=np.zeros((n, 2), bool),
                   starting_stacks=starting_stacks, scale=scale, board=full, bb=bb)

    @classmethod
    def preflop(cls, n: int, starting_stacks=20000, button=0, sb: int = 50, bb: int = 100, scale=None) -> "RootStates":
        """Roots as the environment's reset leaves them (src/p2/env/hunl_tensor_env.py:293-317):
        the button posts the small blind and acts first, the other player the big blind."""
        button = np.broadcast_to(np.asarray(button, dtype=np.int64), (n,)).copy()
        starting_stacks = np.broadcast_to(np.asarray(starting_stacks, dtype=np.int64), (n, 2)).copy()
        committed = np.where(np.arange(2)[None, :] == button[:, None], sb, bb).astype(np.int64)
        if scale is None:
            scale = starting_stacks[:, 0].astype(np.float32)
        scale = np.broadcast_to(np.asarray(scale, dtype=np.float32), (n,)).copy()
        return cls(street=np.zeros(n, np.int64), to_act=button.copy(), button=button,
                   pot=np.full(n, sb + bb, np.int64), stacks=starting_stacks - committed, committed=committed,
                   min_raise=np.full(n, bb, np.int64), actions_this_round=np.zeros(n, np.int64),
                   is_allin=np.zeros((n, 2), bool), starting_stacks=starting_stacks, scale=scale,
                   board=np.full((n, 5), -1, np.int64), bb=bb)

    @classmethod
    def from_env(cls, env, indices) -> "RootStates":
        """Copy rows of an object exposing the reference env's attribute names
        (``HUNLTensorEnv``: button, street, to_act, pot, stacks, committed, min_raise,
        actions_this_round, is_allin, starting_stacks, scale, board_indices, done, bb; optional
        last_board_indices and deck)."""
        if getattr(env, "flop_showdown", False):
            raise NotImplementedError("roots of the env's flop_showdown game variant (hunl_tensor_env.py:900) are not "
                                      "supported: the tree builders follow the full game")
        def g(name):
            x = getattr(env, name)
            x = x.detach().cpu().numpy() if hasattr(x, "detach") else np.asarray(x)
            return x[np.asarray(indices)]
        idx = indices.detach().cpu().numpy() if hasattr(indices, "detach") else np.asarray(indices)
        indices = idx
        return cls(street=g("street").astype(np.int64), to_act=g("to_act").astype(np.int64),
                   button=g("button").astype(np.int64), pot=g("pot").astype(np.int64),
                   stacks=g("stacks").astype(np.int64), committed=g("committed").astype(np.int64),
                   min_raise=g("min_raise").astype(np.int64),
                   actions_this_round=g("actions_this_round").astype(np.int64),
                   is_allin=g("is_allin").astype(bool), starting_stacks=g("starting_stacks").astype(np.int64),
                   scale=g("scale").astype(np.float32), board=g("board_indices").astype(np.int64),
                   done=g("done").astype(bool), bb=int(getattr(env, "bb", 100)),
                   last_board=g("last_board_indices").astype(np.int64) if hasattr(env, "last_board_indices") else None,
                   # the env deals streets from the deck it was reset with: four hole cards, then the five
                   # board cards (hunl_tensor_env.py:280-285, 900-975)
                   runout=g("deck")[:, 4:9].astype(np.int64) if hasattr(env, "deck") else None)


_STATE_FIELDS = ("street", "to_act", "button", "pot", "stacks", "committed", "min_raise", "actions_this_round",
                 "is_allin", "starting_stacks", "scale", "done", "raises")


def _legal_mask(s: dict, bins: list[float], max_raises: int | None) -> tuple[np.ndarray, np.ndarray]:
    n = s["pot"].shape[0]
    nb = len(bins) + 3
    rows = np.arange(n)
    me, opp = s["to_act"], 1 - s["to_act"]
    me_stack, opp_stack = s["stacks"][rows, me], s["stacks"][rows, opp]
    to_call = s["committed"][rows, opp] - s["committed"][rows, me]
    amounts = np.full((n, nb), -1, dtype=np.int64)
    mask = np.zeros((n, nb), dtype=bool)
    mask[:, 0] = to_call > 0
    mask[:, 1] = True
    fr = np.asarray(bins, dtype=np.float32)
    additional = (fr[None, :] * s["pot"].astype(np.float32)[:, None]).astype(np.int64)  # truncates
    amt = to_call[:, None] + additional
    can = (me_stack > 0) & (opp_stack > 0)
    amounts[:, 2:-1] = amt
    mask[:, 2:-1] = can[:, None] & (amt <= me_stack[:, None]) & (additional >= s["min_raise"][:, None])
    amounts[:, nb - 1] = me_stack
    mask[:, nb - 1] = me_stack > 0
    if max_raises is not None:
        capped = s["raises"] >= max_raises
        mask[capped, 2:] = False
    opp_allin = s["is_allin"][rows, opp]
    mask[opp_allin, 0:2] = True
    mask[opp_allin, 2:] = False
    me_allin = s["is_allin"][rows, me]
    mask[me_allin, :] = False
    mask[me_allin, 1] = True
    mask &= ~s["done"][:, None]
    return amounts, mask


def _step(parent: dict, prow: np.ndarray, bins_taken: np.ndarray, amounts: np.ndarray, nb: int, bb: int):
    """Children of ``parent`` rows ``prow`` after taking ``bins_taken``; returns (state, fold reward)."""
    c = {k: parent[k][prow].copy() for k in _STATE_FIELDS}
    m = prow.shape[0]
    rows = np.arange(m)
    me, opp = c["to_act"].copy(), 1 - c["to_act"]
    to_call = c["committed"][rows, opp] - c["committed"][rows, me]
    me_stack = c["stacks"][rows, me]
    fold = bins_taken == 0
    call = bins_taken == 1
    allin = bins_taken == nb - 1
    bet = ~(fold | call | allin)
    chips = np.zeros(m, dtype=np.int64)
    chips[call] = np.minimum(to_call, me_stack)[call]
    chips[allin] = me_stack[allin]
    chips[bet] = amounts[prow, bins_taken][bet]
    c["stacks"][rows, me] -= chips
    c["committed"][rows, me] += chips
    c["pot"] += chips
    c["is_allin"][rows[allin], me[allin]] = True
    c["min_raise"][bet] = np.maximum(c["min_raise"], chips - to_call)[bet]
    c["raises"] = c["raises"] + (bet | allin).astype(np.int64)
    # fold: the other player takes the pot; value for player 0 in units of `scale`
    reward = np.zeros(m, dtype=np.float32)
    f32 = np.float32
    share = np.where(opp == 0, c["pot"].astype(f32), f32(0.0))
    r = (c["stacks"][:, 0].astype(f32) + share - c["starting_stacks"][:, 0].astype(f32)) / c["scale"]
    reward[fold] = r[fold]
    c["done"] = c["done"] | fold
    c["to_act"] = 1 - c["to_act"]
    c["actions_this_round"] = c["actions_this_round"] + 1
    equal = c["committed"][:, 0] == c["committed"][:, 1]
    a0, a1 = c["is_allin"][:, 0], c["is_allin"][:, 1]
    covered = (a0 & a1) | (a0 & (c["committed"][:, 0] <= c["committed"][:, 1])) | \
        (a1 & (c["committed"][:, 1] <= c["committed"][:, 0]))
    closed = ~c["done"] & (equal | covered) & (c["actions_this_round"] >= 2)
    c["committed"][closed] = 0
    c["actions_this_round"][closed] = 0
    c["raises"][closed] = 0
    c["to_act"][closed] = 1 - c["button"][closed]
    c["min_raise"][closed] = bb
    c["done"] = c["done"] | (closed & (c["street"] == 3))  # river closes into a showdown
    c["street"] = c["street"] + closed.astype(np.int64)
    return c, reward


@dataclass
class SparseTree:
    depth_offsets: list
    n_roots: int
    total: int
    num_actions: int
    bet_bins: list
    parent_index: np.ndarray
    action_from_parent: np.ndarray
    child_count: np.ndarray
    child_offsets: np.ndarray
    prev_actor: np.ndarray
    root_index: np.ndarray
    legal_mask: np.ndarray
    leaf_mask: np.ndarray
    new_street_mask: np.ndarray
    fold_mask: np.ndarray
    showdown_mask: np.ndarray
    reward: np.ndarray
    state: dict = field(repr=False)
    board: np.ndarray = None      # [n_roots,5]

    @property
    def tree_depth(self) -> int:
        return max(0, len(self.depth_offsets) - 2)

    @property
    def top(self) -> int:
        return self.depth_offsets[-2] if len(self.depth_offsets) > 1 else self.n_roots

    def __getattr__(self, name):
        st = object.__getattribute__(self, "state")
        if name in st:
            return st[name]
        raise AttributeError(name)

    @property
    def showdown_potential(self) -> np.ndarray:
        """[total,2] chips player p nets by winning the pot (sparse_cfr_evaluator.py:249-253)."""
        return self.state["stacks"] + self.state["pot"][:, None] - self.state["starting_stacks"]


def build_sparse_tree(roots: RootStates, bet_bins: list[float], depth: int,
                      max_raises: int | None = None) -> SparseTree:
    """Breadth-first expansion to ``depth`` plies.  Below the root level a node whose betting
    round has just closed (``actions_this_round == 0``, which includes showdowns) is not
    expanded (sparse_cfr_evaluator.py:167-197)."""
    _req(roots.n > 0, "must supply at least one root state")
    bins = [float(b) for b in bet_bins]
    nb = len(bins) + 3
    n = roots.n
    s0 = {k: np.array(getattr(roots, k)) for k in _STATE_FIELDS if k != "raises"}
    s0["raises"] = np.zeros(n, dtype=np.int64)
    levels = [s0]
    parents = [np.full(n, -1, dtype=np.int64)]
    actions = [np.full(n, -1, dtype=np.int64)]
    rewards = [np.zeros(n, dtype=np.float32)]
    offsets = [0, n]
    d = 0
    while d < depth:
        par = levels[-1]
        amounts, legal = _legal_mask(par, bins, max_raises)
        if d > 0:
            legal &= (par["actions_this_round"] != 0)[:, None]
        prow, taken = np.nonzero(legal)  # parent-major, action-ascending
        if prow.size == 0:
            break
        child, rew = _step(par, prow, taken, amounts, nb, roots.bb)
        levels.append(child)
        parents.append(prow + offsets[-2])
        actions.append(taken.astype(np.int64))
        rewards.append(rew)
        offsets.append(offsets[-1] + prow.size)
        d += 1
    state = {k: np.concatenate([lv[k] for lv in levels]) for k in _STATE_FIELDS}
    total = offsets[-1]
    parent_index = np.concatenate(parents)
    action = np.concatenate(actions)
    reward = np.concatenate(rewards)
    _, legal = _legal_mask(state, bins, max_raises)
    is_root = np.zeros(total, dtype=bool)
    is_root[:n] = True
    new_street = (state["actions_this_round"] == 0) & ~is_root
    leaf = state["done"] | new_street
    leaf[offsets[-2]:] = True
    child_mask = legal & ~leaf[:, None]
    child_count = child_mask.sum(axis=1).astype(np.int64)
    _req(total == n + int(child_count.sum()), "total == n + int(child_count.sum())")
    _req((child_count[~leaf] > 0).all() and not leaf[:n].any(),
         "(child_count[~leaf] > 0).all() and not leaf[:n].any()")
    child_offsets = (offsets[1] + np.cumsum(child_count) - child_count).astype(np.int64)
    prev_actor = np.full(total, -1, dtype=np.int64)
    prev_actor[n:] = state["to_act"][parent_index[n:]]
    root_index = np.arange(total, dtype=np.int64)
    for lv in range(len(offsets) - 2):
        s, e = offsets[lv + 1], offsets[lv + 2]
        root_index[s:e] = root_index[parent_index[s:e]]
    return SparseTree(depth_offsets=list(offsets), n_roots=n, total=total, num_actions=nb, bet_bins=bins,
                      parent_index=parent_index, action_from_parent=action, child_count=child_count,
                      child_offsets=child_offsets, prev_actor=prev_actor, root_index=root_index,
                      legal_mask=legal, leaf_mask=leaf, new_street_mask=new_street,
                      fold_mask=(action == 0) & state["done"], showdown_mask=state["street"] == 4,
                      reward=reward, state=state, board=np.array(roots.board))


# Items that start in the last rounds of a launch are started largest first; three rounds of the 768
# workgroups an MI355X holds at a time (3 per compute unit x 256).
SORTED_TAIL_ITEMS = 3 * 768


def launch_order(size: np.ndarray, sorted_tail: int = SORTED_TAIL_ITEMS) -> np.ndarray:
    """Order in which work items of the given sizes are handed to the compute units: ascending index —
    items that run at the same time then work on neighbouring rows of every tensor, which the memory
    system rewards (4096 three-raise roots: 11.2 ms per iteration with all items sorted by size, 10.3 ms
    this way) — except that the last ``sorted_tail`` items come largest first: a launch lasts until its last
    item ends, so the long ones must not be the ones that start last.  A launch of fewer items than that is
    sorted by size as a whole."""
    n = len(size)
    order = np.arange(n)
    w = min(int(sorted_tail), n)
    if w > 0:
        tail = order[n - w:]
        order = np.concatenate([order[:n - w], tail[np.argsort(-np.asarray(size)[tail], kind="stable")]])
    return order.astype(np.int64)


def split_work_items(tree: "SparseTree", n_roots: int, cut_level: int, mid_level=None,
                     sorted_tail: int = SORTED_TAIL_ITEMS):
    """Work items for the iteration kernel when a root gets several workgroups (include/p2hip.h), in
    tiers: tier 0 holds one item per root, the top of its tree above the first cut level; every further
    tier one item per node of its cut level that has children, with the families from that level down
    to the next cut level (the last tier: to the leaves).  Cut levels: ``mid_level`` (optional: one level or
    several, those above the main one count) and ``cut_level``.  On three-raise river trees a cut at
    level 1 and one at level 2 measured best; further cuts at levels 3 and 4 make items smaller and
    iterations 3-30 % slower (4096 to 192 roots), each tier costing two more launches.  Returns numpy arrays over all items in tier order (family
    rows + offsets, showdown rows + offsets, item_root, item_top) and the tiers' item counts; None if
    the tree is too shallow to cut."""
    N, T = n_roots, tree.total
    offs = tree.depth_offsets
    n_levels = len(offs) - 1
    has_children = tree.child_count > 0
    cut = min(cut_level, n_levels - 2)
    while cut >= 1 and not has_children[offs[cut]:offs[cut + 1]].any():
        cut -= 1                                            # the deepest level that still has families below it
    if cut < 1:
        return None
    mids = [] if mid_level is None else ([mid_level] if np.isscalar(mid_level) else list(mid_level))
    cuts = sorted({int(m) for m in mids if 1 <= m < cut}) + [cut]

    def grouped(rows, keys, groups):
        """rows ordered by group (ascending inside a group) and offsets [len(groups) + 1]."""
        slot = np.searchsorted(groups, keys)
        order = np.argsort(slot, kind="stable")
        counts = np.bincount(slot, minlength=len(groups))
        return rows[order], np.concatenate([[0], np.cumsum(counts)])

    def reordered(rows, offsets, order):
        pieces = [rows[offsets[g]:offsets[g + 1]] for g in order]
        lengths = np.array([len(x) for x in pieces], dtype=np.int64)
        return (np.concatenate(pieces) if pieces else rows), np.concatenate([[0], np.cumsum(lengths)])
    roots = np.arange(N)
    # tier 0: families whose parent lies above the first cut, showdown rows down to that cut, per root
    upper = np.nonzero(has_children[:offs[cuts[0]]])[0]
    lists_p = [grouped(upper, tree.root_index[upper], roots)]
    upper_sd = np.nonzero(tree.showdown_mask[:offs[cuts[0] + 1]])[0]
    lists_s = [grouped(upper_sd, tree.root_index[upper_sd], roots)]
    item_root, item_top, tiers = [roots], [np.ones(N, np.uint8)], [N]
    for j, lo in enumerate(cuts):
        hi = cuts[j + 1] if j + 1 < len(cuts) else n_levels          # parent levels lo .. hi-1
        anchor = np.full(T, -1, dtype=np.int64)    # the level-`lo` node a deeper row sits under (itself there)
        anchor[offs[lo]:offs[lo + 1]] = np.arange(offs[lo], offs[lo + 1])
        for d in range(lo + 1, n_levels):
            rows = np.arange(offs[d], offs[d + 1])
            anchor[rows] = anchor[tree.parent_index[rows]]
        heads = np.nonzero(has_children[offs[lo]:offs[lo + 1]])[0] + offs[lo]        # ascending rows
        span = np.arange(offs[lo], offs[hi] if hi < n_levels else T)
        parent_rows = span[has_children[span]]
        tp, tpo = grouped(parent_rows, anchor[parent_rows], heads)
        sd_rows = np.arange(offs[lo + 1], offs[hi + 1] if hi < n_levels else T)
        sd_rows = sd_rows[tree.showdown_mask[sd_rows]]
        sd_rows = sd_rows[np.isin(anchor[sd_rows], heads)]
        ts, tso = grouped(sd_rows, anchor[sd_rows], heads)
        below = np.arange(offs[lo], offs[hi + 1] if hi < n_levels else T)
        below = below[np.isin(anchor[below], heads)]
        size = np.bincount(np.searchsorted(heads, anchor[below]), minlength=len(heads))
        order = launch_order(size, sorted_tail)
        lists_p.append(reordered(tp, tpo, order))
        lists_s.append(reordered(ts, tso, order))
        heads = heads[order]
        item_root.append(tree.root_index[heads])
        item_top.append(np.zeros(len(heads), np.uint8))
        tiers.append(len(heads))

    def joined(lists):
        rows = np.concatenate([r for r, _ in lists]).astype(np.int64)
        offsets, base = [np.zeros(1, np.int64)], 0
        for _, o in lists:
            offsets.append(base + o[1:])
            base += o[-1]
        return rows, np.concatenate(offsets).astype(np.int64)
    parents, parent_offsets = joined(lists_p)
    showdown, showdown_offsets = joined(lists_s)
    _req(len(parents) == int(has_children.sum()) and len(showdown) == int(tree.showdown_mask.sum()),
         "every family and every showdown row must belong to exactly one work item")
    return SimpleNamespace(parents=parents, parent_offsets=parent_offsets, showdown=showdown,
                           showdown_offsets=showdown_offsets, item_root=np.concatenate(item_root).astype(np.int64),
                           item_top=np.concatenate(item_top), tiers=tiers, n_sub=sum(tiers[1:]), cut=cut, cuts=cuts)


# ---------------------------------------------------------------------------------------------
# Device builder: the same tree, expanded by two HIP kernels per level.
_DEVICE_COLS = ("street", "to_act", "button", "pot", "stack0", "stack1", "comm0", "comm1", "min_raise",
                "actions_this_round", "allin0", "allin1", "start0", "start1", "done", "raises", "scale", "root",
                "parent", "action", "reward")


def build_sparse_tree_device(roots: RootStates, bet_bins: list[float], depth: int,
                             max_raises: int | None = None, device="cuda") -> SparseTree:
    """``build_sparse_tree`` on the GPU (``p2hip_tree_legal`` / ``p2hip_tree_step``): identical
    arrays, bit for bit.  The returned tree also carries ``device_arrays`` — the index arrays as
    resident torch tensors — so the evaluator does not upload them again.  One small
    device-to-host read per level (the number of children) and one copy of the finished node
    table back to the host."""
    import ctypes

    import torch

    from . import _lib
    if not _lib.hip_is_available():
        raise RuntimeError("build_sparse_tree_device needs libp2hip.so and a GPU; use build_sparse_tree on the host.")
    _req(roots.n > 0, "must supply at least one root state")
    bins = [float(b) for b in bet_bins]
    if len(bins) > 5:
        raise ValueError("at most 5 bet fractions (8 action bins) are supported")
    nb = len(bins) + 3
    n = roots.n
    dev = torch.device(device)
    cols = int(_lib.load().p2hip_tree_node_columns())
    _req(cols == len(_DEVICE_COLS), "cols == len(_DEVICE_COLS)")
    host = np.zeros((n, cols), dtype=np.int64)
    col = {name: i for i, name in enumerate(_DEVICE_COLS)}
    for name in ("street", "to_act", "button", "pot", "min_raise", "actions_this_round", "done"):
        host[:, col[name]] = np.asarray(getattr(roots, name)).astype(np.int64)
    for name, src in (("stack", roots.stacks), ("comm", roots.committed), ("allin", roots.is_allin),
                      ("start", roots.starting_stacks)):
        host[:, col[name + "0"]] = np.asarray(src)[:, 0].astype(np.int64)
        host[:, col[name + "1"]] = np.asarray(src)[:, 1].astype(np.int64)
    host[:, col["scale"]] = np.asarray(roots.scale, dtype=np.float32).view(np.uint32).astype(np.int64)
    host[:, col["root"]] = np.arange(n)
    host[:, col["parent"]] = -1
    host[:, col["action"]] = -1
    bins_c = (ctypes.c_float * max(1, len(bins)))(*bins)
    bins_p = ctypes.cast(bins_c, ctypes.c_void_p)
    mr = -1 if max_raises is None else int(max_raises)
    levels = [torch.from_numpy(host).to(dev)]
    legal_l, count_l = [], []
    offsets = [0, n]
    d = 0
    while True:
        cur = levels[-1]
        k = cur.shape[0]
        expand = d < depth
        legal = torch.empty(k, nb, dtype=torch.uint8, device=dev)
        count = torch.empty(k, dtype=torch.int64, device=dev)
        _lib.call("p2hip_tree_legal", _lib.ptr(cur), k, bins_p, len(bins), mr, int(d == 0), int(expand),
                  _lib.ptr(legal), _lib.ptr(count), _lib.stream_ptr())
        legal_l.append(legal)
        count_l.append(count)
        if not expand:
            break
        ends = torch.cumsum(count, 0)
        n_next = int(ends[-1].item())
        if n_next == 0:
            break
        start = (ends - count).contiguous()
        child = torch.empty(n_next, cols, dtype=torch.int64, device=dev)
        _lib.call("p2hip_tree_step", _lib.ptr(cur), k, int(offsets[-2]), bins_p, len(bins), mr, int(roots.bb),
                  int(d == 0), _lib.ptr(start), _lib.ptr(child), _lib.stream_ptr())
        levels.append(child)
        offsets.append(offsets[-1] + n_next)
        d += 1
    nodes = torch.cat(levels) if len(levels) > 1 else levels[0]
    legal = torch.cat(legal_l).bool()
    child_count = torch.cat(count_l)
    total = offsets[-1]
    child_offsets = (n + torch.cumsum(child_count, 0) - child_count).contiguous()
    # the one bulk copy back to the host, column-major so that every column is a contiguous row
    columns = nodes.t().contiguous()
    table = columns.cpu().numpy()

    def c(name):
        return table[col[name]]
    state = {
        "street": c("street"), "to_act": c("to_act"), "button": c("button"), "pot": c("pot"),
        "stacks": np.stack([c("stack0"), c("stack1")], axis=1),
        "committed": np.stack([c("comm0"), c("comm1")], axis=1),
        "min_raise": c("min_raise"), "actions_this_round": c("actions_this_round"),
        "is_allin": np.stack([c("allin0"), c("allin1")], axis=1).astype(bool),
        "starting_stacks": np.stack([c("start0"), c("start1")], axis=1),
        "scale": c("scale").astype(np.uint32).view(np.float32), "done": c("done").astype(bool), "raises": c("raises"),
    }
    parent_index, action = c("parent"), c("action")
    reward = c("reward").astype(np.uint32).view(np.float32)
    is_root = np.zeros(total, dtype=bool)
    is_root[:n] = True
    new_street = (state["actions_this_round"] == 0) & ~is_root
    leaf = state["done"] | new_street
    leaf[offsets[-2]:] = True
    cc = child_count.cpu().numpy()
    _req(total == n + int(cc.sum()), "total == n + int(cc.sum())")
    prev_actor = np.full(total, -1, dtype=np.int64)
    prev_actor[n:] = state["to_act"][parent_index[n:]]
    tree = SparseTree(depth_offsets=list(offsets), n_roots=n, total=total, num_actions=nb, bet_bins=bins,
                      parent_index=parent_index, action_from_parent=action, child_count=cc,
                      child_offsets=child_offsets.cpu().numpy(), prev_actor=prev_actor, root_index=c("root"),
                      legal_mask=legal.cpu().numpy(), leaf_mask=leaf, new_street_mask=new_street,
                      fold_mask=(action == 0) & state["done"], showdown_mask=state["street"] == 4,
                      reward=reward, state=state, board=np.array(roots.board))
    object.__setattr__(tree, "device_arrays", {
        "parent_index": columns[col["parent"]], "action_from_parent": columns[col["action"]],
        "child_count": child_count, "child_offsets": child_offsets, "root_index": columns[col["root"]],
        "legal_mask": legal, "to_act": columns[col["to_act"]], "street": columns[col["street"]],
        "pot": columns[col["pot"]], "button": columns[col["button"]],
        "actions_this_round": columns[col["actions_this_round"]], "min_raise": columns[col["min_raise"]],
        "stacks": torch.stack([columns[col["stack0"]], columns[col["stack1"]]], dim=1),
        "committed": torch.stack([columns[col["comm0"]], columns[col["comm1"]]], dim=1),
        "starting_stacks": torch.stack([columns[col["start0"]], columns[col["start1"]]], dim=1),
        "is_allin": torch.stack([columns[col["allin0"]], columns[col["allin1"]]], dim=1).bool(),
        "done": columns[col["done"]].bool(),
        "scale": columns[col["scale"]].to(torch.int32).view(torch.float32),
        "reward": columns[col["reward"]].to(torch.int32).view(torch.float32),
    })
    # masks the evaluator keeps on the device, derived there instead of copied back
    d_done = tree.device_arrays["done"]
    d_new_street = (columns[col["actions_this_round"]] == 0)
    d_new_street[:n] = False
    d_leaf = d_done | d_new_street
    d_leaf[offsets[-2]:] = True
    d_prev = torch.full((total,), -1, dtype=torch.int64, device=dev)
    d_prev[n:] = columns[col["to_act"]][columns[col["parent"]][n:]]
    d_pot = tree.device_arrays["stacks"] + columns[col["pot"]][:, None] - tree.device_arrays["starting_stacks"]
    tree.device_arrays.update({
        "new_street_mask": d_new_street, "leaf_mask": d_leaf, "prev_actor": d_prev,
        "fold_mask": (columns[col["action"]] == 0) & d_done, "showdown_mask": columns[col["street"]] == 4,
        "showdown_potential": d_pot,
    })
    return tree
