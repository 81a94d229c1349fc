"""Combo indexing, blocker masks and unblocked mass with the reference's names.

Mirrors the in-scope part of ``src/p2/env/card_utils.py`` (:58-149, :196-222):
the integer tables are built once on the host and cached per device;
``calculate_unblocked_mass`` runs the HIP kernel (GPU tensors only, no CPU path).
"""
from __future__ import annotations

from functools import lru_cache

import torch

from . import _lib

NUM_HANDS = 1326


@lru_cache(maxsize=8)
def hand_combos_tensor(device: torch.device | None = None) -> torch.Tensor:
    """[1326, 2] int64 rows (c1 < c2), lexicographic (card_utils.py:58-68)."""
    c1, c2 = torch.triu_indices(52, 52, offset=1)
    t = torch.stack([c1, c2], dim=1).to(torch.long)
    return t if device is None else t.to(device)


@lru_cache(maxsize=8)
def combo_lookup_tensor(device: torch.device | None = None) -> torch.Tensor:
    """[52, 52] int64 symmetric lookup, -1 on the diagonal (card_utils.py:71-81)."""
    combos = hand_combos_tensor()
    lut = torch.full((52, 52), -1, dtype=torch.long)
    idx = torch.arange(NUM_HANDS)
    lut[combos[:, 0], combos[:, 1]] = idx
    lut[combos[:, 1], combos[:, 0]] = idx
    return lut if device is None else lut.to(device)


def combo_index(card_a: int, card_b: int) -> int:
    """Index of the unordered pair; ValueError for equal cards (card_utils.py:84-91)."""
    a, b = sorted((int(card_a), int(card_b)))
    if a == b or a < 0 or b > 51:
        raise ValueError(f"Invalid combo for cards {card_a}, {card_b}")
    return a * (103 - a) // 2 + (b - a - 1)


def mask_conflicting_combos(occupied_cards: torch.Tensor, device: torch.device | None = None) -> torch.Tensor:
    """[1326] bool, True = combo shares no card with ``occupied_cards`` (-1 ignored)
    (card_utils.py:94-111)."""
    combos = hand_combos_tensor(device=device)
    occupied = occupied_cards[occupied_cards >= 0]
    if occupied.numel() == 0:
        return torch.ones(combos.shape[0], dtype=torch.bool, device=device)
    return ~torch.isin(combos, occupied.to(combos.device)).any(dim=1)


@lru_cache(maxsize=8)
def combo_to_onehot_tensor(device: torch.device | None = None) -> torch.Tensor:
    """[1326, 52] bool (card_utils.py:114-122)."""
    combos = hand_combos_tensor()
    oh = torch.zeros(NUM_HANDS, 52, dtype=torch.bool)
    idx = torch.arange(NUM_HANDS)
    oh[idx, combos[:, 0]] = True
    oh[idx, combos[:, 1]] = True
    return oh if device is None else oh.to(device)


@lru_cache(maxsize=4)
def combo_blocking_tensor(device: torch.device | None = None) -> torch.Tensor:
    """[1326, 1326] bool, True where two combos share a card (card_utils.py:138-142)."""
    oh = combo_to_onehot_tensor().to(torch.int16)
    out = (oh @ oh.T) > 0
    return out if device is None else out.to(device)


@lru_cache(maxsize=4)
def combo_compatible_tensor(device: torch.device | None = None) -> torch.Tensor:
    """Complement of the blocking tensor; a combo is not compatible with itself
    (card_utils.py:145-149)."""
    out = ~combo_blocking_tensor()
    return out if device is None else out.to(device)


def suit_permutations_tensor(device: torch.device | None = None) -> torch.Tensor:
    """[24, 4] int64: every permutation of the four suits, lexicographic (card_utils.py:153-158)."""
    from itertools import permutations
    perms = torch.tensor(tuple(permutations(range(4))), dtype=torch.long)
    return perms if device is None else perms.to(device)


@lru_cache(maxsize=8)
def combo_suit_permutation_tensor(device: torch.device | None = None) -> torch.Tensor:
    """[24, 1326] int64: index of the combo each combo becomes when the suits are permuted
    (card_utils.py:161-181)."""
    combos = hand_combos_tensor()
    ranks, suits = combos % 13, combos // 13
    cards = suit_permutations_tensor()[:, suits] * 13 + ranks[None]          # [24, 1326, 2]
    lo, hi = cards.min(dim=2).values, cards.max(dim=2).values
    out = combo_lookup_tensor()[lo, hi]
    return out if device is None else out.to(device)


@lru_cache(maxsize=8)
def combo_suit_permutation_inverse_tensor(device: torch.device | None = None) -> torch.Tensor:
    """[24, 1326] int64: argsort of ``combo_suit_permutation_tensor`` per row (card_utils.py:184-193)."""
    inv = torch.argsort(combo_suit_permutation_tensor(), dim=1)
    return inv if device is None else inv.to(device)


def calculate_unblocked_mass(target: torch.Tensor) -> torch.Tensor:
    """[..., 1326] -> same shape: mass of the combos sharing no card with each combo,
    clamped at 0 (card_utils.py:196-222).  Runs ``p2hip_unblocked_mass``."""
    _lib.require_gpu(target, "calculate_unblocked_mass")
    if target.shape[-1] != NUM_HANDS:
        raise ValueError(f"last dim must be {NUM_HANDS}, got {tuple(target.shape)}")
    flat = target.reshape(-1, NUM_HANDS).contiguous().float()
    out = torch.empty_like(flat)
    _lib.call("p2hip_unblocked_mass", _lib.ptr(flat), flat.shape[0], _lib.ptr(out), _lib.stream_ptr())
    return out.view(target.shape)
