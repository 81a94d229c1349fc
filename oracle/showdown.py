"""River showdown EV with card-blocker correction.  TEST INFRASTRUCTURE ONLY.

Follows ``src/p2/search/cfr_evaluator.py``:
  init_hand_rank_data   <- _init_hand_rank_data   :406-482
  showdown_value        <- _showdown_value        :492-601
  showdown_value_both   <- _showdown_value_both   :484-490
and, as the brute-force check, the enumeration in the reference's
``tests/test_rebel_cfr_evaluator.py:294-338`` (showdown_value_bruteforce).

The villain range is gathered into strength order, prefix-summed globally and
per card (the [M,1327,52] tensor of the reference), and for a hero hand with
cards (c1,c2) whose tie group spans sorted positions [L,R):
  win  = P[L] - Pc[L,c1] - Pc[L,c2]
  tie  = (P[R]-P[L]) - (Pc[R,c1]-Pc[L,c1]) - (Pc[R,c2]-Pc[L,c2]) + b_self
  den  = max(1 - Pc[end,c1] - Pc[end,c2] + b_self, 1e-8)
  EV   = win/den - (1 - win/den - tie/den)      (0 where den <= 1e-8)
then un-sorted, zeroed on board-blocked hands and scaled by potential/scale.
Prefix sums accumulate in float64 and are rounded to float32 per element, which
is what torch's CPU cumsum does for float32 input.

Pinned by: brute force over all hero x villain pairs (several boards from the
reference's tests), all-tie board -> 0, delta villain -> +-potential,
zero-sum identity over compatible pairs, |EV| <= potential/scale; and by outputs of the
reference's own ``showdown_ev_triton`` kernel (fused_cfr_triton.py:2162-2314) run under Triton's
CPU interpreter (tests/golden/fused_ops_golden.npz, case ``showdown_sorted``).  The formula takes
the villain range as normalised and zero on board-blocked hands (the constant 1 in
``den``), as the evaluator guarantees; it is not invariant to rescaling the range.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from .cards import NUM_HANDS, combo_blocking, combo_onehot, hand_combos, mask_conflicting
from .ranker import rank_hands


@dataclass
class HandRankData:
    sorted_indices: np.ndarray   # [M,H] int64, weakest -> strongest (stable)
    inv_sorted: np.ndarray       # [M,H] int64
    card_ok: np.ndarray          # [M,52] bool, False on board cards
    hand_ok_mask: np.ndarray     # [M,H] bool
    hands_c1c2_sorted: np.ndarray  # [M,H,2] int64
    L_idx: np.ndarray            # [M,H] int32 first sorted position of the tie group
    R_idx: np.ndarray            # [M,H] int32 one past the last


def init_hand_rank_data(board: np.ndarray, hand_ok_mask: np.ndarray,
                        ranker=rank_hands) -> HandRankData:
    board = np.asarray(board, dtype=np.int64)
    m = board.shape[0]
    hand_ranks, order = ranker(board)
    ranks_sorted = np.take_along_axis(hand_ranks, order, axis=1)
    assert (ranks_sorted[:, 1:] >= ranks_sorted[:, :-1]).all()
    is_start = np.ones_like(ranks_sorted, dtype=bool)
    is_start[:, 1:] = ranks_sorted[:, 1:] != ranks_sorted[:, :-1]
    gid = np.cumsum(is_start, axis=1) - 1
    k = np.broadcast_to(np.arange(NUM_HANDS), (m, NUM_HANDS))
    starts = np.full((m, NUM_HANDS), NUM_HANDS, dtype=np.int64)
    ends = np.full((m, NUM_HANDS), -1, dtype=np.int64)
    rows = np.broadcast_to(np.arange(m)[:, None], (m, NUM_HANDS))
    np.minimum.at(starts, (rows, gid), k)
    np.maximum.at(ends, (rows, gid), k)
    L = np.take_along_axis(starts, gid, axis=1)
    R = np.take_along_axis(ends, gid, axis=1)
    inv = np.argsort(order, axis=1, kind="stable")
    card_ok = np.ones((m, 52), dtype=bool)
    card_ok[np.arange(m)[:, None], board] = False
    c1c2 = hand_combos()[order]  # [M,H,2]
    return HandRankData(
        sorted_indices=order.astype(np.int64),
        inv_sorted=inv.astype(np.int64),
        card_ok=card_ok,
        hand_ok_mask=np.asarray(hand_ok_mask, dtype=bool),
        hands_c1c2_sorted=c1c2,
        L_idx=L.astype(np.int32),
        R_idx=np.minimum(R + 1, NUM_HANDS).astype(np.int32),
    )


def _cumsum_f32(x: np.ndarray, axis: int) -> np.ndarray:
    return np.cumsum(x.astype(np.float64), axis=axis).astype(np.float32)


def showdown_value(beliefs: np.ndarray, hero: int, hrd: HandRankData,
                   potential: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """beliefs [M,2,H] float32 -> [M,H] float32 EV of ``hero`` per hand.
    potential [M,2] (chips), scale [M] float32."""
    beliefs = np.asarray(beliefs, dtype=np.float32)
    m = beliefs.shape[0]
    if m == 0:
        return np.zeros((0, NUM_HANDS), dtype=np.float32)
    f32 = np.float32
    b_opp = beliefs[:, 1 - hero, :]
    order = hrd.sorted_indices
    b_sorted = np.take_along_axis(b_opp, order, axis=1)
    c1 = hrd.hands_c1c2_sorted[..., 0]
    c2 = hrd.hands_c1c2_sorted[..., 1]
    onehot_sorted = combo_onehot()[order] & hrd.card_ok[:, None, :]  # [M,H,52]

    P = np.concatenate([np.zeros((m, 1), f32), _cumsum_f32(b_sorted, 1)], axis=1)
    per_card = onehot_sorted.astype(f32) * b_sorted[..., None]
    Pc = np.concatenate([np.zeros((m, 1, 52), f32), _cumsum_f32(per_card, 1)], axis=1)

    L = hrd.L_idx.astype(np.int64)
    R = hrd.R_idx.astype(np.int64)
    rows = np.arange(m)[:, None]
    P_L = np.take_along_axis(P, L, axis=1)
    P_R = np.take_along_axis(P, R, axis=1)
    PcL1 = Pc[rows, L, c1]
    PcL2 = Pc[rows, L, c2]
    PcR1 = Pc[rows, R, c1]
    PcR2 = Pc[rows, R, c2]
    win = P_L - PcL1 - PcL2
    tie = (P_R - P_L) - (PcR1 - PcL1) - (PcR2 - PcL2) + b_sorted
    last = Pc[:, -1, :]
    den = np.maximum(
        f32(1.0) - np.take_along_axis(last, c1, axis=1) - np.take_along_axis(last, c2, axis=1) + b_sorted,
        f32(1e-8),
    )
    valid = den > f32(1e-8)
    win_p = np.where(valid, win / den, f32(0.0))
    tie_p = np.where(valid, tie / den, f32(0.0))
    loss_p = np.where(valid, f32(1.0) - win_p - tie_p, f32(0.0))
    ev_sorted = (win_p - loss_p).astype(f32)
    ev = np.take_along_axis(ev_sorted, hrd.inv_sorted, axis=1)
    ev = ev * hrd.hand_ok_mask.astype(f32)
    pot = np.asarray(potential)[:, hero].astype(f32)
    return (ev * pot[:, None] / np.asarray(scale, dtype=f32)[:, None]).astype(f32)


def showdown_value_both(beliefs, hrd, potential, scale) -> np.ndarray:
    out = np.empty_like(np.asarray(beliefs, dtype=np.float32))
    out[:, 0] = showdown_value(beliefs, 0, hrd, potential, scale)
    out[:, 1] = showdown_value(beliefs, 1, hrd, potential, scale)
    return out


def showdown_value_bruteforce(board, opp_beliefs, potential: float,
                              ranker=rank_hands) -> np.ndarray:
    """Enumerate every (hero, villain) pair on one board in float64.
    EV[h] = potential * (P(win | compatible villain) - P(lose | ...))."""
    board = np.asarray(board, dtype=np.int64)
    ok = mask_conflicting(board)
    opp = np.asarray(opp_beliefs, dtype=np.float64) * ok
    opp = opp / max(opp.sum(), 1e-12)
    ranks = ranker(board[None])[0][0]
    blocking = combo_blocking()
    ev = np.zeros(NUM_HANDS)
    for h in np.nonzero(ok)[0]:
        compat = (~blocking[h]) & ok
        cond = opp * compat
        tot = cond.sum()
        if tot <= 0:
            continue
        cond = cond / tot
        ev[h] = potential * ((cond * (ranks < ranks[h])).sum() - (cond * (ranks > ranks[h])).sum())
    return ev
