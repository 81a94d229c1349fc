"""Chance nodes around the leaf network (one card; the three-card flop).  TEST INFRASTRUCTURE ONLY.

Follows ``ChanceNodeHelper.single_card_chance_values``
(src/p2/search/chance_node_helper.py:360-479):
  expand   :394-443  every (state, card not on its board) sample, state-major and card
                     ascending; the card goes into the first empty board slot; ranges lose the
                     hands that touch the sample's board and are renormalised per player
                     (uniform over the allowed hands where the sum is <= 1e-12)
  model    :445-465  the network sees (context, street, to_act) of the state, the sample's
                     board and the flattened post-chance ranges
  mean     :467-477  sum of the network's hand values per state / number of its samples; the
                     hands that hold the dealt card are NOT excluded from the mean

Pinned by vectors written from the reference's own helper (tests/golden/chance_golden.npz,
made by tests/golden/gen_chance_golden.py: echo and board-and-range networks, mixed turn / flop
boards, dead and delta ranges) and by (tests/test_oracle_chance.py) a per-sample Python loop written from the docstring
above, closed forms for an echo network (mean of the renormalised ranges), a board-only
network (mean over cards of a function of the board), sample counts 52 - k, and the
reference's own empty / shape cases (tests/test_chance_node_helper.py:426-478).

Three-card chance node, ``ChanceNodeHelper.flop_chance_values`` (:219-357) with its canonical
flop cache (:76-216) and the suit maps of src/p2/env/card_utils.py:153-193:
  canonical_flops      per flop, a Python loop over the 24 suit permutations; the smallest
                       base-52 code of (cards by rank descending, equal ranks' suits ascending)
  combo_suit_perms     [24,1326] hand index after each suit permutation
  flop_expand          ranges lose the hands touching the flop, renormalised (uniform over the
                       1176 left if dead)
  flop_chance_values   enumeration weighted by class size / 22100, or the plain mean over a given
                       sample of class ids; each flop's answer is the mean over the given
                       permutations of hv[..., perm[h]]
Pinned by tests/golden/flop_chance_golden.npz (tests/golden/gen_flop_chance_golden.py runs the
reference's helper: the cache tables, an exhaustive all-permutation pass and seeded sampled passes
for networks that depend on board suits and hand index) and by closed forms in
tests/test_oracle_chance.py (class sizes sum to 22100 and follow the rank pattern; a
suit-equivariant network gives the plain mean over all 22100 flops).
"""
from __future__ import annotations

import numpy as np

from .cards import NUM_HANDS, combo_lookup, combo_onehot, hand_combos


def expand(pre_beliefs: np.ndarray, board_prev: np.ndarray):
    """pre_beliefs [B,2,H] float32, board_prev [B,5] int64 (-1 = empty).
    Returns post_beliefs [S,2,H] float32, board_samples [S,5], root_lookup [S]."""
    pre_beliefs = np.asarray(pre_beliefs, dtype=np.float32)
    board_prev = np.asarray(board_prev, dtype=np.int64)
    b = pre_beliefs.shape[0]
    available = np.ones((b, 52), dtype=bool)
    for slot in range(board_prev.shape[1]):
        cards = board_prev[:, slot]
        valid = cards >= 0
        available[np.nonzero(valid)[0], cards[valid]] = False
    flat = np.nonzero(available.reshape(-1))[0]
    root_lookup = flat // 52
    card_values = flat % 52
    s = flat.size
    board_samples = board_prev[root_lookup].copy()
    num_cards = (board_samples >= 0).sum(axis=1)
    board_samples[np.arange(s), num_cards] = card_values
    board_onehot = np.zeros((s, 52), dtype=bool)
    i_s, i_slot = np.nonzero(board_samples >= 0)
    board_onehot[i_s, board_samples[i_s, i_slot]] = True
    allowed = (combo_onehot().astype(np.float32) @ board_onehot.T.astype(np.float32) < 0.5).T   # [S,H]
    post = pre_beliefs[root_lookup].copy()
    post[np.broadcast_to(~allowed[:, None, :], post.shape)] = 0.0
    sums = post.sum(axis=-1, keepdims=True, dtype=np.float32)
    uniform = allowed[:, None, :].astype(np.float32)
    uniform = uniform / np.maximum(uniform.sum(axis=-1, keepdims=True), np.float32(1.0))
    post = np.where(sums > np.float32(1e-12), post / np.maximum(sums, np.float32(1e-12)), uniform)
    return post.astype(np.float32), board_samples, root_lookup


def mean_by_root(hand_values: np.ndarray, root_lookup: np.ndarray, b: int) -> np.ndarray:
    hand_values = np.asarray(hand_values, dtype=np.float32)
    values_sum = np.zeros((b, 2, NUM_HANDS), dtype=np.float32)
    np.add.at(values_sum, root_lookup, hand_values)
    counts = np.maximum(np.bincount(root_lookup, minlength=b).astype(np.float32), np.float32(1.0))
    return (values_sum / counts[:, None, None]).astype(np.float32)


def single_card_chance_values(root_indices, context, street, to_act, pre_chance_beliefs, board_pre, model_fn):
    """``model_fn(context[S,C], street[S], to_act[S], board[S,5], beliefs[S,2*H]) -> [S,2,H]``."""
    root_indices = np.asarray(root_indices, dtype=np.int64)
    if root_indices.size == 0:
        return np.zeros((0, 2, NUM_HANDS), dtype=np.float32)
    b = root_indices.size
    post, board_samples, root_lookup = expand(np.asarray(pre_chance_beliefs)[root_indices],
                                              np.asarray(board_pre)[root_indices])
    if root_lookup.size == 0:
        return np.zeros((b, 2, NUM_HANDS), dtype=np.float32)
    src = root_indices[root_lookup]
    hv = model_fn(np.asarray(context)[src], np.asarray(street)[src], np.asarray(to_act)[src], board_samples,
                  post.reshape(post.shape[0], -1))
    return mean_by_root(hv, root_lookup, b)


# ---- three-card (flop) chance node --------------------------------------------------------

def suit_permutations() -> np.ndarray:
    """[24,4]: permutations of (0,1,2,3) in lexicographic order (card_utils.py:153-158)."""
    from itertools import permutations
    return np.array(list(permutations(range(4))), dtype=np.int64)


def combo_suit_perms() -> np.ndarray:
    """[24,1326]: index of hand h once every card's suit s becomes perm[s] (card_utils.py:161-181)."""
    combos, lookup, perms = hand_combos(), combo_lookup(), suit_permutations()
    out = np.zeros((perms.shape[0], NUM_HANDS), dtype=np.int64)
    for q, perm in enumerate(perms):
        for h, (a, b) in enumerate(combos):
            x, y = perm[a // 13] * 13 + a % 13, perm[b // 13] * 13 + b % 13
            out[q, h] = lookup[min(x, y), max(x, y)]
    return out


def canonical_flops():
    """(canonical [K,3], count [K], flop_to_class [22100]) following chance_node_helper.py:76-216."""
    from itertools import combinations
    perms = suit_permutations()
    best_codes = []
    for flop in combinations(range(52), 3):
        by_rank = sorted(flop, key=lambda c: -(c % 13))
        ranks = [c % 13 for c in by_rank]
        best = None
        for perm in perms:
            suits = [int(perm[c // 13]) for c in by_rank]
            if ranks[0] == ranks[1] == ranks[2]:
                suits = sorted(suits)
            elif ranks[0] == ranks[1]:
                suits[:2] = sorted(suits[:2])
            elif ranks[1] == ranks[2]:
                suits[1:] = sorted(suits[1:])
            cards = [s_ * 13 + r for s_, r in zip(suits, ranks)]
            code = cards[0] * 2704 + cards[1] * 52 + cards[2]
            best = code if best is None or code < best else best
        best_codes.append(best)
    codes = np.array(best_codes, dtype=np.int64)
    unique, flop_to_class = np.unique(codes, return_inverse=True)
    canonical = np.stack([unique // 2704, (unique // 52) % 52, unique % 52], axis=1)
    count = np.bincount(flop_to_class, minlength=unique.size).astype(np.int64)
    return canonical, count, flop_to_class.astype(np.int64)


def flop_expand(pre_beliefs: np.ndarray, flops: np.ndarray) -> np.ndarray:
    """pre_beliefs [B,2,H], flops [K,3] -> [B,K,2,H] (chance_node_helper.py:268-286)."""
    pre_beliefs = np.asarray(pre_beliefs, dtype=np.float32)
    onehot = combo_onehot().astype(np.float32)                                   # [H,52]
    board = np.zeros((flops.shape[0], 52), dtype=np.float32)
    for k, f in enumerate(flops):
        board[k, f] = 1.0
    allowed = (onehot @ board.T == 0).T                                           # [K,H]
    post = np.repeat(pre_beliefs[:, None], flops.shape[0], axis=1)
    post[np.broadcast_to(~allowed[None, :, None, :], post.shape)] = 0.0
    sums = post.sum(axis=-1, keepdims=True, dtype=np.float32)
    uniform = allowed[None, :, None, :].astype(np.float32)
    uniform = uniform / np.maximum(uniform.sum(axis=-1, keepdims=True), np.float32(1.0))
    return np.where(sums > np.float32(1e-12), post / np.maximum(sums, np.float32(1e-12)), uniform).astype(np.float32)


def flop_chance_values(root_indices, context, street, to_act, pre_chance_beliefs, model_fn, canonical, count,
                       combo_perm, sample_idx=None, perm_rows=None, chunk=128):
    """Enumeration (sample_idx None: weights count / sum(count)) or plain mean over the classes
    in sample_idx.  perm_rows: list, per chunk, of the rows of combo_perm to average (None = all).
    ``model_fn`` as in single_card_chance_values (chance_node_helper.py:219-357)."""
    root_indices = np.asarray(root_indices, dtype=np.int64)
    b = root_indices.size
    if b == 0:
        return np.zeros((0, 2, NUM_HANDS), dtype=np.float32)
    pre = np.asarray(pre_chance_beliefs, dtype=np.float32)[root_indices]
    ctx, st, ta = np.asarray(context)[root_indices], np.asarray(street)[root_indices], np.asarray(to_act)[root_indices]

    def eval_chunk(flops, rows):
        k = flops.shape[0]
        post = flop_expand(pre, flops)
        board5 = np.concatenate([flops, np.full((k, 2), -1, dtype=np.int64)], axis=1)
        hv = model_fn(np.repeat(ctx, k, axis=0), np.repeat(st, k), np.repeat(ta, k), np.tile(board5, (b, 1)),
                      post.reshape(b * k, -1)).reshape(b, k, 2, NUM_HANDS).astype(np.float32)
        perms = combo_perm if rows is None else combo_perm[np.asarray(rows)]
        return np.mean(np.stack([hv[..., q] for q in perms], axis=0, dtype=np.float64), axis=0)   # [B,k,2,H]

    if sample_idx is not None:
        rows = None if perm_rows is None else perm_rows[0]
        return eval_chunk(canonical[np.asarray(sample_idx)], rows).mean(axis=1).astype(np.float32)
    total = np.zeros((b, 2, NUM_HANDS), dtype=np.float64)
    for j, start in enumerate(range(0, canonical.shape[0], chunk)):
        end = min(start + chunk, canonical.shape[0])
        rows = None if perm_rows is None else perm_rows[j]
        total += (eval_chunk(canonical[start:end], rows) * count[start:end, None, None][None]).sum(axis=1)
    return (total / float(count.sum())).astype(np.float32)
