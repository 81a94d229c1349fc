"""7-card hand ranker (numpy restatement).  TEST INFRASTRUCTURE ONLY.

Follows ``src/p2/env/rules.py``:
  comparison_fields   <- create_comparison_vector   :136-299
  pack_fields         <- nibble packing             :111-112, :406-407
  compare_planes      <- compare_7_single_batch     :390-409
  rank_hands          <- rank_hands                 :66-133
and ``src/p2/env/rules_triton.py``:
  rank_cards          <- _evaluate_cards_player     :414-581  (card-id input;
                         a duplicated card id counts again towards
                         pairs/trips/quads, and carries into the next bit of
                         its suit's mask, which is a SUM of rank bits)
  rank_hands_cards    <- rank_hands_triton          :120-148

Card encoding: card = suit*13 + rank, rank 0..12 = 2..A.

Field semantics (all deliberately reproduce the reference, including where
it is not standard poker):
  * ranks are ordered by (count desc, rank desc); the five leading entries
    ``i0..i4`` feed every count-based category; absent ranks (count 0) pad
    the list high -> low;
  * straight flush [9, highest window]; quads [8, i0, i1]; full house
    [7, i0, i1] iff cnt0>=3 and cnt1>=2; flush [6, top five ranks of the
    flush suit]; straight [5, LOWEST qualifying window]; trips [4,i0,i1,i2];
    two pair [3,i0,i1,i2]; pair [2,i0..i3]; high card [1,i0..i4];
  * window w in 0..9 covers ranks w-1..w+3 with the ace doubling as rank -1.

Pinned by: (1) ``tests/golden/ranker_golden.npz`` -- packed scores written by
running the reference's own ``rules.py`` in the build container on 4096 seeded
random hands plus targeted quirk hands (quads+pair, three pairs, 6/7-card
runs, wheel+six, short hands); (2) the 45 ordered hand pairs and three
rank-order lists of the reference's ``tests/test_rules.py`` (restated as data in
``tests/golden/rules_pairs.json``); (3) the exhaustive C(52,7) category
histogram equalling the textbook table; (4) agreement with an independent
best-5-of-7 evaluator (``oracle/std_eval.c``) outside the quirk classes.

(5) for hands that REPEAT a card id (which ``rules.py`` cannot express and ``rank_hands_triton``
produces for every combo that holds a board card): ``tests/golden/ranker_cards_golden.npz`` -- scores
written by running the reference's own card-id kernel under Triton's CPU interpreter on 316 such
hands and on all 1326 combos of three boards (``tests/golden/gen_ranker_cards_golden.py``; its two
PTX leaf helpers, highest set bit and population count, are replaced there by plain integer code of
the same meaning).
"""
from __future__ import annotations

import numpy as np

from .cards import NUM_HANDS, hand_combos

_RANKS = np.arange(13, dtype=np.int32)
_WINDOWS = np.arange(10, dtype=np.int32)


def cards_to_planes(cards: np.ndarray) -> np.ndarray:
    """[..., K] card ids (negative = no card) -> [..., 4, 13] bool planes."""
    cards = np.asarray(cards, dtype=np.int64)
    lead = cards.shape[:-1]
    flat = cards.reshape(-1, cards.shape[-1])
    planes = np.zeros((flat.shape[0], 52), dtype=bool)
    rows = np.arange(flat.shape[0])
    for j in range(flat.shape[1]):
        ok = flat[:, j] >= 0
        planes[rows[ok], flat[ok, j]] = True
    return planes.reshape(*lead, 4, 13)


def _sliding5(x: np.ndarray) -> np.ndarray:
    """Sum over windows of 5 along the last axis: [...,14] -> [...,10]."""
    return x[..., 0:10] + x[..., 1:11] + x[..., 2:12] + x[..., 3:13] + x[..., 4:14]


def comparison_fields(planes: np.ndarray) -> np.ndarray:
    """[..., 4, 13] 0/1 planes -> [..., 6] int32 (type, five kicker fields)."""
    planes = np.asarray(planes).astype(np.int32)
    lead = planes.shape[:-2]
    rank_sum = planes.sum(axis=-2)  # [...,13]
    key = (rank_sum << 8) | _RANKS
    # five largest keys, descending (keys are distinct, so the order is total)
    order = np.argsort(-key, axis=-1, kind="stable")[..., :5]
    top_idx = order.astype(np.int32)
    top_cnt = np.take_along_axis(rank_sum, order, axis=-1)

    table = np.zeros(lead + (10, 6), dtype=np.int32)

    # straight flush: any suit with five in a window; highest such window
    ext = np.concatenate([planes[..., 12:13], planes], axis=-1)  # [...,4,14]
    sf_win = (_sliding5(ext).max(axis=-2) == 5)  # [...,10]
    has_sf = sf_win.any(axis=-1)
    sf_last = (sf_win.astype(np.int32) * _WINDOWS).max(axis=-1)
    table[..., 9, 0] = np.where(has_sf, 9, 0)
    table[..., 9, 1] = np.where(has_sf, sf_last, -1)

    c0, c1 = top_cnt[..., 0], top_cnt[..., 1]
    quads = c0 >= 4
    table[..., 8, 0] = np.where(quads, 8, 0)
    table[..., 8, 1:3] = np.where(quads[..., None], top_idx[..., :2], 0)

    full = (c0 >= 3) & (c1 >= 2)
    table[..., 7, 0] = np.where(full, 7, 0)
    table[..., 7, 1:3] = np.where(full[..., None], top_idx[..., :2], 0)

    # flush: suit with the most cards (first on ties) must hold >= 5
    suit_sum = planes.sum(axis=-1)  # [...,4]
    flush = suit_sum.max(axis=-1) >= 5
    fsuit = suit_sum.argmax(axis=-1)
    suit_cards = np.take_along_axis(planes, fsuit[..., None, None], axis=-2)[..., 0, :]
    scores = np.where(suit_cards > 0, _RANKS, -1)
    top5 = -np.sort(-scores, axis=-1)[..., :5]
    table[..., 6, 0] = np.where(flush, 6, 0)
    table[..., 6, 1:6] = np.where(flush[..., None], top5, 0)

    # straight: lowest window whose five ranks are all present
    presence = np.clip(ext.sum(axis=-2), 0, 1)  # [...,14]
    conv = _sliding5(presence)
    straight = conv.max(axis=-1) == 5
    low = conv.argmax(axis=-1)
    table[..., 5, 0] = np.where(straight, 5, 0)
    table[..., 5, 1] = np.where(straight, low, 0)

    trips = c0 >= 3
    table[..., 4, 0] = np.where(trips, 4, 0)
    table[..., 4, 1:4] = np.where(trips[..., None], top_idx[..., :3], 0)

    two_pair = (c0 >= 2) & (c1 >= 2)
    table[..., 3, 0] = np.where(two_pair, 3, 0)
    table[..., 3, 1:4] = np.where(two_pair[..., None], top_idx[..., :3], 0)

    pair = c0 >= 2
    table[..., 2, 0] = np.where(pair, 2, 0)
    table[..., 2, 1:5] = np.where(pair[..., None], top_idx[..., :4], 0)

    table[..., 1, 0] = 1
    table[..., 1, 1:6] = top_idx

    best = table[..., 0].argmax(axis=-1)
    return np.take_along_axis(table, best[..., None, None], axis=-2)[..., 0, :]


def pack_fields(fields: np.ndarray) -> np.ndarray:
    """[..., 6] -> [...] int32, field i shifted left by 4*(5-i), summed."""
    shifts = 4 * (5 - np.arange(6, dtype=np.int32))
    return (np.asarray(fields, dtype=np.int32) << shifts).sum(axis=-1).astype(np.int32)


def rank_planes(planes: np.ndarray) -> np.ndarray:
    """Packed int32 score per hand from [..., 4, 13] planes."""
    return pack_fields(comparison_fields(planes))


def compare_planes(ab: np.ndarray) -> np.ndarray:
    """[N, 2, 4, 13] -> [N] int32 in {-1, 0, 1} (1 = first hand wins)."""
    packed = rank_planes(ab)
    return np.clip(packed[:, 0] - packed[:, 1], -1, 1).astype(np.int32)


def _popcount(x: np.ndarray) -> np.ndarray:
    x = x.astype(np.int64)
    return sum((x >> k) & 1 for k in range(32)).astype(np.int32)


def _highest_bit(x: np.ndarray) -> np.ndarray:
    """Index of the most significant set bit, 0 for an empty mask (``_pop_highest_rank``,
    rules_triton.py:364-375: ``bfind`` clamped at 0)."""
    x = x.astype(np.int64)
    return sum(((x >> k) != 0).astype(np.int32) for k in range(1, 32)).astype(np.int32)


def rank_cards(cards: np.ndarray) -> np.ndarray:
    """Packed int32 score from card ids [..., K] as ``_evaluate_cards_player`` scores them
    (rules_triton.py:414-581): a repeated id counts again towards the rank multiplicities
    (:431-440), and each suit's mask is the integer SUM of its cards' rank bits (``tl.sum``,
    :421-425), so a repeated card carries into the next higher bit of its suit's mask; straights
    come from the ranks present; the flush suit is the first suit whose mask has >= 5 bits, its
    five kickers the mask's highest bits; straight-flush windows look at bits 0..12 of the masks."""
    cards = np.asarray(cards, dtype=np.int64)
    lead = cards.shape[:-1]
    flat = cards.reshape(-1, cards.shape[-1])
    n = flat.shape[0]
    rows = np.arange(n)
    ranks = flat % 13
    suits = flat // 13
    counts = np.zeros((n, 13), dtype=np.int32)
    suit_mask = np.zeros((n, 4), dtype=np.int64)
    for j in range(flat.shape[1]):
        np.add.at(counts, (rows, ranks[:, j]), 1)
        np.add.at(suit_mask, (rows, suits[:, j]), np.int64(1) << ranks[:, j])
    counts = np.minimum(counts, 4)

    key = (counts << 8) | _RANKS
    order = np.argsort(-key, axis=-1, kind="stable")[:, :5]
    top_idx = order.astype(np.int32)
    top_cnt = np.take_along_axis(counts, order, axis=-1)
    c0, c1 = top_cnt[:, 0], top_cnt[:, 1]

    def pk(t, *f):
        f = list(f) + [0] * (5 - len(f))
        val = np.asarray(t, dtype=np.int32) << 20
        for i, x in enumerate(f):
            val = val | (np.asarray(x, dtype=np.int32) << (4 * (4 - i)))
        return val

    suit_planes = ((suit_mask[:, :, None] >> _RANKS.astype(np.int64)) & 1).astype(np.int32)   # bits 0..12 of the masks
    ext = np.concatenate([suit_planes[..., 12:13], suit_planes], axis=-1)
    sf_win = _sliding5(ext).max(axis=-2) == 5
    has_sf = sf_win.any(axis=-1)
    sf_high = (sf_win.astype(np.int32) * _WINDOWS).max(axis=-1)
    presence = np.clip(counts, 0, 1)
    pext = np.concatenate([presence[:, 12:13], presence], axis=-1)
    conv = _sliding5(pext)
    straight = conv.max(axis=-1) == 5
    low = conv.argmax(axis=-1)

    has5 = _popcount(suit_mask) >= 5
    flush = has5.any(axis=-1)
    fsuit = np.where(flush, has5.argmax(axis=-1), 3)
    remaining = suit_mask[rows, fsuit]
    fl = []
    for _ in range(5):
        best = _highest_bit(remaining)
        fl.append(best)
        remaining = remaining & ~(np.int64(1) << best.astype(np.int64))

    z = np.zeros(n, dtype=np.int32)
    w = np.where
    scores = [
        pk(1, *[top_idx[:, i] for i in range(5)]),
        w(c0 >= 2, pk(2, *[top_idx[:, i] for i in range(4)]), z),
        w((c0 >= 2) & (c1 >= 2), pk(3, *[top_idx[:, i] for i in range(3)]), z),
        w(c0 >= 3, pk(4, *[top_idx[:, i] for i in range(3)]), z),
        w(straight, pk(5, low), z),
        w(flush, pk(6, *fl), z),
        w((c0 >= 3) & (c1 >= 2), pk(7, top_idx[:, 0], top_idx[:, 1]), z),
        w(c0 >= 4, pk(8, top_idx[:, 0], top_idx[:, 1]), z),
        w(has_sf, pk(9, sf_high), z),
    ]
    out = scores[0]
    for s in scores[1:]:
        out = np.maximum(out, s)
    return out.astype(np.int32).reshape(lead)


def _dense_ranks(packed: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    order = np.argsort(packed, axis=1, kind="stable")
    sp = np.take_along_axis(packed, order, axis=1)
    start = np.ones_like(sp, dtype=np.int32)
    start[:, 1:] = (sp[:, 1:] != sp[:, :-1]).astype(np.int32)
    gid = np.cumsum(start, axis=1, dtype=np.int32)
    out = np.zeros_like(gid)
    np.put_along_axis(out, order, gid, axis=1)
    return out, order.astype(np.int64)


def rank_hands(board: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """All 1326 combos on each board [M,5].

    Returns (dense 1-based group ids [M,1326] int32, stable ascending argsort
    [M,1326] int64).  A combo sharing a card with the board is evaluated on the
    union of its planes with the board's, i.e. as a 6-card hand
    (``rules.py:89-102``)."""
    board = np.asarray(board, dtype=np.int64)
    m = board.shape[0]
    combos = hand_combos()
    planes = np.zeros((m, NUM_HANDS, 52), dtype=bool)
    planes[:, np.arange(NUM_HANDS), combos[:, 0]] = True
    planes[:, np.arange(NUM_HANDS), combos[:, 1]] = True
    bp = np.zeros((m, 52), dtype=bool)
    bp[np.arange(m)[:, None], board] = True
    planes |= bp[:, None, :]
    packed = rank_planes(planes.reshape(m, NUM_HANDS, 4, 13))
    return _dense_ranks(packed)


def rank_hands_cards(board: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """Card-id variant: returns (packed scores [M,1326] int32, stable argsort);
    hole cards first, then the board (``rules_triton.py:139-148``)."""
    board = np.asarray(board, dtype=np.int64)
    m = board.shape[0]
    combos = hand_combos()
    cards = np.concatenate(
        [np.broadcast_to(combos[None], (m, NUM_HANDS, 2)),
         np.broadcast_to(board[:, None, :], (m, NUM_HANDS, 5))], axis=-1)
    packed = rank_cards(cards)
    order = np.argsort(packed, axis=1, kind="stable").astype(np.int64)
    return packed, order
