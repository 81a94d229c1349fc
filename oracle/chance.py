"""Single-card chance node around the leaf network.  TEST INFRASTRUCTURE ONLY.

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
"""
from __future__ import annotations

import numpy as np

from .cards import NUM_HANDS, combo_onehot


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
