"""Unblocked (card-compatible) mass.  TEST INFRASTRUCTURE ONLY.

  calculate_unblocked_mass   <- src/p2/env/card_utils.py:196-222
        out[h] = sum over h' sharing no card with h of t[h'], computed as a
        float64 product with the 1326x1326 compatibility matrix, cast to
        float32, clamped at 0.  A combo blocks itself (diagonal 0).
  unblocked_mass_inclusion_exclusion
                             <- src/p2/search/fused_cfr_triton.py:928-959,
                                :1008-1026, :1110-1157
        S - cardsum[a] - cardsum[b] + t[h] with S and the 52 card sums taken in
        float32, clamped at 0.
  unblocked_mass_ratio       <- fused_cfr_triton.py:1408-1496 (K12):
        denom > eps ? unblk(numer)/unblk(denom) : 0

Pinned by the reference's known answers (tests/test_card_utils.py:472-614:
uniform -> 1225/1326 = 0.9238311052322388, delta -> 0 on itself and its
blockers and 1 elsewhere, two half deltas -> 0.5 ...), by the identity of the
two formulations, by an explicit double loop on a few rows, and by outputs of the
reference's own unblocked-mass kernels (plain, opponent-at-parents, ratio direct
and indirect) run under Triton's CPU interpreter (tests/golden/fused_ops_golden.npz,
tests/test_oracle_fused_ops.py).
"""
from __future__ import annotations

import numpy as np

from .cards import NUM_HANDS, combo_compatible, combo_onehot, hand_combos


def calculate_unblocked_mass(target: np.ndarray) -> np.ndarray:
    t = np.asarray(target, dtype=np.float32)
    flat = t.reshape(-1, NUM_HANDS).astype(np.float64)
    out = (flat @ combo_compatible().astype(np.float64)).astype(np.float32)
    return np.maximum(out.reshape(t.shape), np.float32(0.0))


def card_stats(target: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """(S [B], cardsum [B,52]) in float32 for a [B,1326] float32 input."""
    t = np.asarray(target, dtype=np.float32).reshape(-1, NUM_HANDS)
    s = t.sum(axis=-1, dtype=np.float32)
    cs = t @ combo_onehot().astype(np.float32)
    return s, cs.astype(np.float32)


def unblocked_mass_inclusion_exclusion(target: np.ndarray) -> np.ndarray:
    t = np.asarray(target, dtype=np.float32)
    flat = t.reshape(-1, NUM_HANDS)
    s, cs = card_stats(flat)
    cm = hand_combos()
    out = s[:, None] - cs[:, cm[:, 0]] - cs[:, cm[:, 1]] + flat
    return np.maximum(out, np.float32(0.0)).reshape(t.shape).astype(np.float32)


def unblocked_mass_ratio(numer: np.ndarray, denom: np.ndarray, eps: float = 1e-5,
                         parent_index: np.ndarray | None = None) -> np.ndarray:
    """``parent_index`` (optional) gathers the denominator row per numerator
    row, as the indirect kernel does (fused_cfr_triton.py:1408-1453)."""
    n = calculate_unblocked_mass(numer)
    d = calculate_unblocked_mass(denom)
    if parent_index is not None:
        d = d[np.asarray(parent_index)]
    safe = np.where(d > np.float32(eps), d, np.float32(1.0))
    return np.where(d > np.float32(eps), n / safe, np.float32(0.0)).astype(np.float32)


def unblocked_mass_loops(row: np.ndarray) -> np.ndarray:
    """Explicit O(H^2) double loop in float64 for one row (brute force)."""
    row = np.asarray(row, dtype=np.float64)
    cm = hand_combos()
    out = np.zeros(NUM_HANDS)
    for i in range(NUM_HANDS):
        a, b = cm[i]
        ok = (cm[:, 0] != a) & (cm[:, 0] != b) & (cm[:, 1] != a) & (cm[:, 1] != b)
        out[i] = row[ok].sum()
    return out
