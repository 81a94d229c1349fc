"""CPU: pins the oracle's card tables and ranker (numpy + C) against the reference-held
vectors, the golden fixtures, closed forms and an independent textbook evaluator."""
import json
import os

import numpy as np
import pytest

from oracle import cards as OC
from oracle import ranker as R
from oracle import ranker_c as RC
from tests.helpers import C


def test_combo_indexing_known_answers():
    # reference tests/test_card_utils.py:44-47, :96-104, :118-128
    assert OC.combo_index(0, 1) == 0 and OC.combo_index(0, 2) == 1
    assert OC.combo_index(1, 2) == 51 and OC.combo_index(50, 51) == 1325
    assert OC.combo_index(2, 1) == 51
    with pytest.raises(ValueError):
        OC.combo_index(5, 5)
    cm = OC.hand_combos()
    assert cm.shape == (1326, 2) and (cm[:, 0] < cm[:, 1]).all()
    a, b = cm[:, 0], cm[:, 1]
    assert np.array_equal(a * (103 - a) // 2 + (b - a - 1), np.arange(1326))
    lut = OC.combo_lookup()
    assert (np.diag(lut) == -1).all() and np.array_equal(lut, lut.T)
    assert np.array_equal(lut[a, b], np.arange(1326))


def test_blocker_tables():
    oh = OC.combo_onehot()
    assert oh.sum(axis=1).tolist() == [2] * 1326 and oh.sum(axis=0).tolist() == [51] * 52
    blk = OC.combo_blocking()
    assert blk.diagonal().all() and np.array_equal(blk, blk.T)
    assert (blk.sum(axis=1) == 101).all()  # 51 + 51 - 1
    assert np.array_equal(OC.combo_compatible(), ~blk)
    for k, expect in ((5, 1081), (4, 1128), (3, 1176), (0, 1326)):
        board = np.full((1, 5), -1)
        board[0, :k] = np.arange(k) * 7
        allowed, prob = OC.allowed_hands_for_boards(board)
        assert allowed.sum() == expect
        np.testing.assert_allclose(prob.sum(), 1.0, rtol=1e-6)
        assert np.array_equal(allowed[0], OC.mask_conflicting(board[0]))


def test_ranker_golden_vectors(golden_dir):
    g = np.load(os.path.join(golden_dir, "ranker_golden.npz"))
    cards = g["cards"].astype(np.int64)
    planes = R.cards_to_planes(cards)
    assert np.array_equal(R.comparison_fields(planes), g["fields"].astype(np.int32))
    assert np.array_equal(R.rank_planes(planes), g["packed"])
    assert np.array_equal(RC.rank_planes(planes), g["packed"])
    full = (cards >= 0).all(axis=1)
    assert np.array_equal(R.rank_cards(cards[full]), g["packed"][full])
    assert np.array_equal(RC.rank_cards(cards), g["packed"])  # C skips absent (-1) cards
    ab = np.stack([planes[:-1], planes[1:]], axis=1)
    assert np.array_equal(R.compare_planes(ab), g["cmp_adjacent"].astype(np.int32))
    ranks, order = R.rank_hands(g["boards"].astype(np.int64))
    assert np.array_equal(ranks, g["board_ranks"].astype(np.int32))
    assert np.array_equal(order, g["board_order"].astype(np.int64))


def test_reference_test_pairs(golden_dir):
    with open(os.path.join(golden_dir, "rules_pairs.json")) as f:
        pairs = json.load(f)["pairs"]
    assert len(pairs) >= 35
    for p in pairs:
        sa = RC.rank_planes(R.cards_to_planes(np.array([p["a"]])))[0]
        sb = RC.rank_planes(R.cards_to_planes(np.array([p["b"]])))[0]
        assert int(np.sign(int(sa) - int(sb))) == p["expected"], p["test"]


def test_rank_order_lists_of_reference_tests():
    # tests/test_rules.py:530-607 -- strongest to weakest hole cards on two boards
    board1 = np.array([[C(8, 0), C(8, 1), C(8, 2), C(0, 0), C(1, 0)]])
    tc = C(8, 3)
    holes1 = [(tc, C(12, 1)), (tc, C(11, 2)), (tc, C(10, 3)), (tc, C(9, 3)), (tc, C(3, 1)),
              (C(12, 0), C(12, 3)), (C(11, 0), C(11, 3)), (C(12, 0), C(2, 0)), (C(11, 0), C(2, 0)),
              (C(10, 0), C(2, 0)), (C(9, 0), C(2, 0)), (C(7, 0), C(2, 0)), (C(12, 1), C(11, 0)),
              (C(12, 0), C(7, 3)), (C(5, 1), C(3, 1))]
    board2 = np.array([[C(1, 1), C(2, 1), C(3, 1), C(7, 2), C(12, 2)]])
    holes2 = [(C(9, 1), C(12, 1)), (C(6, 1), C(9, 1)), (C(4, 0), C(5, 2)), (C(0, 2), C(6, 3)),
              (C(7, 0), C(7, 3)), (C(12, 0), C(3, 2)), (C(12, 3), C(11, 2)), (C(12, 3), C(6, 2)),
              (C(7, 0), C(6, 2)), (C(11, 0), C(10, 3)), (C(8, 3), C(6, 0)), (C(6, 0), C(5, 0))]
    for board, holes in ((board1, holes1), (board2, holes2)):
        ranks = R.rank_hands(board)[0][0]
        vals = [ranks[OC.combo_index(a, b)] for a, b in holes]
        assert all(x > y for x, y in zip(vals, vals[1:]))
        packed = R.rank_hands_cards(board)[0][0]
        vals = [packed[OC.combo_index(a, b)] for a, b in holes]
        assert all(x > y for x, y in zip(vals, vals[1:]))


def test_exhaustive_category_histogram():
    hist = RC.hist_all7()
    assert hist.sum() == 133784560
    assert [int(x) for x in hist] == [0, 23294460, 58627800, 31433400, 6461620, 6180020, 4047644, 3473184,
                                      224848, 41584]


def _quirk_mask(cards: np.ndarray) -> np.ndarray:
    """Hands in the classes where the reference departs from standard poker kickers."""
    ranks = cards % 13
    cnt = np.zeros((cards.shape[0], 13), dtype=np.int32)
    np.add.at(cnt, (np.repeat(np.arange(cards.shape[0]), 7), ranks.reshape(-1)), 1)
    quads_with_pair = (cnt == 4).any(1) & ((cnt == 2) | (cnt == 3)).any(1)
    three_pairs = (cnt == 2).sum(1) == 3
    pres = (cnt > 0).astype(np.int32)
    ext = np.concatenate([pres[:, 12:13], pres], axis=1)
    win = sum(ext[:, i:i + 10] for i in range(5)) == 5
    multi_straight = win.sum(1) > 1
    return quads_with_pair | three_pairs | multi_straight


def test_agrees_with_textbook_evaluator_outside_quirk_classes():
    rng = np.random.default_rng(1)
    cards = np.argsort(rng.random((300000, 52)), axis=1)[:, :7]
    a = RC.rank_cards(cards).astype(np.int64)
    s = RC.std_best5(cards).astype(np.int64)
    assert np.array_equal(a >> 20, s >> 20)  # categories are standard everywhere
    ok = ~_quirk_mask(cards)
    a, s = a[ok], s[ok]
    o = np.argsort(s, kind="stable")
    a, s = a[o], s[o]
    # same order and same ties as the textbook evaluator
    assert np.array_equal(np.sign(np.diff(a)), np.sign(np.diff(s)))


def test_numpy_and_c_oracles_agree_on_random_and_short_hands():
    rng = np.random.default_rng(2)
    cards = np.argsort(rng.random((20000, 52)), axis=1)[:, :7]
    assert np.array_equal(R.rank_cards(cards), RC.rank_cards(cards))
    assert np.array_equal(R.rank_planes(R.cards_to_planes(cards)), RC.rank_cards(cards))
    dup = cards.copy()
    dup[:, 1] = dup[:, 0]
    assert np.array_equal(R.rank_cards(dup), RC.rank_cards(dup))
    short = cards.copy()
    short[:, 4:] = -1
    assert np.array_equal(R.rank_planes(R.cards_to_planes(short)), RC.rank_cards(short))


def test_repeated_card_ids_match_the_reference_kernel(golden_dir):
    """tests/golden/ranker_cards_golden.npz: scores of the reference's own card-id kernel (run under
    Triton's CPU interpreter) for 316 hands that repeat a card id, 64 that do not, and all 1326 combos of
    three boards through the card assembly of rank_hands_triton.  Both oracles, bit for bit."""
    g = np.load(os.path.join(golden_dir, "ranker_cards_golden.npz"))
    hands, scores = g["hands"], g["scores"]
    assert np.array_equal(R.rank_cards(hands.astype(np.int64)), scores)
    assert np.array_equal(RC.rank_cards(hands), scores)
    packed, order = R.rank_hands_cards(g["boards"])
    assert np.array_equal(packed, g["hand_ranks"]) and np.array_equal(order, g["sorted_indices"])
    # the carry is what the fixture is about: with the suit masks OR-ed instead of summed a third of the hands differ
    sorted_h = np.sort(hands, axis=1)
    assert int((sorted_h[:, 1:] == sorted_h[:, :-1]).any(axis=1).sum()) == 316
