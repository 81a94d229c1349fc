"""Combo indexing and blocker tables (numpy restatement).

Follows ``src/p2/env/card_utils.py``:
  hand_combos          <- hand_combos_tensor          :58-68
  combo_lookup         <- combo_lookup_tensor         :71-81
  combo_index          <- combo_index                 :84-91
  mask_conflicting     <- mask_conflicting_combos     :94-111
  combo_onehot         <- combo_to_onehot_tensor      :114-122
  combo_blocking       <- combo_blocking_tensor       :138-142
  combo_compatible     <- combo_compatible_tensor     :145-149
and the per-root board mask of ``src/p2/search/cfr_evaluator.py:811-815``
(allowed_hands / allowed_hands_prob).

Pinned by: the known answers of the reference's ``tests/test_card_utils.py``
(:44-47, :96-104, :118-128), the triangular closed form
``index(a,b) = a*(103-a)/2 + (b-a-1)``, "every card is in exactly 51 combos",
and C(52-k,2) allowed combos for a k-card board (tests/test_oracle_cards.py).
Card encoding: card = suit*13 + rank, rank 0..12 = 2..A
(``src/p2/env/rules.py:11``).
"""
from __future__ import annotations

import functools

import numpy as np

NUM_HANDS = 1326
NUM_CARDS = 52


@functools.lru_cache(maxsize=None)
def hand_combos() -> np.ndarray:
    """[1326, 2] int64, rows (c1 < c2) in lexicographic order."""
    out = np.empty((NUM_HANDS, 2), dtype=np.int64)
    k = 0
    for c1 in range(NUM_CARDS):
        for c2 in range(c1 + 1, NUM_CARDS):
            out[k, 0] = c1
            out[k, 1] = c2
            k += 1
    assert k == NUM_HANDS
    out.setflags(write=False)
    return out


@functools.lru_cache(maxsize=None)
def combo_lookup() -> np.ndarray:
    """[52, 52] int64 symmetric, -1 on the diagonal."""
    lut = np.full((NUM_CARDS, NUM_CARDS), -1, dtype=np.int64)
    cm = hand_combos()
    idx = np.arange(NUM_HANDS)
    lut[cm[:, 0], cm[:, 1]] = idx
    lut[cm[:, 1], cm[:, 0]] = idx
    lut.setflags(write=False)
    return lut


def combo_index(card_a: int, card_b: int) -> int:
    a, b = sorted((int(card_a), int(card_b)))
    idx = int(combo_lookup()[a, b])
    if idx < 0:
        raise ValueError(f"Invalid combo for cards {card_a}, {card_b}")
    return idx


def mask_conflicting(occupied_cards) -> np.ndarray:
    """[1326] bool, True where the combo shares no card with ``occupied_cards``
    (entries < 0 are ignored)."""
    occ = np.asarray(occupied_cards, dtype=np.int64).reshape(-1)
    occ = occ[occ >= 0]
    cm = hand_combos()
    if occ.size == 0:
        return np.ones(NUM_HANDS, dtype=bool)
    return ~np.isin(cm, occ).any(axis=1)


@functools.lru_cache(maxsize=None)
def combo_onehot() -> np.ndarray:
    """[1326, 52] bool."""
    oh = np.zeros((NUM_HANDS, NUM_CARDS), dtype=bool)
    cm = hand_combos()
    idx = np.arange(NUM_HANDS)
    oh[idx, cm[:, 0]] = True
    oh[idx, cm[:, 1]] = True
    oh.setflags(write=False)
    return oh


@functools.lru_cache(maxsize=None)
def combo_blocking() -> np.ndarray:
    """[1326, 1326] bool, True where two combos share a card (self blocks self)."""
    oh = combo_onehot().astype(np.float32)
    out = (oh @ oh.T) > 0.5
    out.setflags(write=False)
    return out


@functools.lru_cache(maxsize=None)
def combo_compatible() -> np.ndarray:
    out = ~combo_blocking()
    out.setflags(write=False)
    return out


def allowed_hands_for_boards(boards) -> tuple[np.ndarray, np.ndarray]:
    """Per-board mask of combos disjoint from the board and the uniform
    probability over them.

    boards: [N, k] int (entries < 0 = card not dealt).
    Returns (allowed [N,1326] bool, allowed_prob [N,1326] float32) as
    ``cfr_evaluator.py:811-815`` builds them: ``(onehot @ board_mask) < 0.5``
    and ``mask / max(mask.sum(), 1)``.
    """
    boards = np.asarray(boards, dtype=np.int64)
    n = boards.shape[0]
    board_mask = np.zeros((n, NUM_CARDS), dtype=np.float32)
    for j in range(boards.shape[1]):
        col = boards[:, j]
        ok = col >= 0
        board_mask[np.nonzero(ok)[0], col[ok]] = 1.0
    allowed = (combo_onehot().astype(np.float32) @ board_mask.T).T < 0.5
    prob = allowed.astype(np.float32)
    prob = prob / np.maximum(prob.sum(axis=-1, keepdims=True), np.float32(1.0))
    return allowed, prob.astype(np.float32)
