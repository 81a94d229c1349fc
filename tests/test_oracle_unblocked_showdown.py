"""CPU: pins the oracle's unblocked-mass and river-showdown restatements.

Unblocked mass: the known answers of the reference's tests/test_card_utils.py:472-614
(uniform 0.92383..., delta, double half delta, the 1326x1326 compatibility product), an O(H^2)
double loop, and the agreement of the GEMM form with the inclusion-exclusion form.
Showdown: enumeration over every hero x villain pair (tests/test_rebel_cfr_evaluator.py:294-338)
on the boards the reference's showdown tests use, plus the cases those tests spell out (sure
win, sure loss, all-tie board) and properties that hold for any input.
"""
import numpy as np
import pytest

from oracle import cards as OC
from oracle import showdown as OS
from oracle import unblocked as OU
from tests.helpers import C, parse_board, random_boards, random_ranges

H = 1326


# ---- unblocked mass -----------------------------------------------------------------------
def test_unblocked_uniform_known_answer():
    u = OU.calculate_unblocked_mass(np.full((1, H), 1.0 / H, np.float32))
    np.testing.assert_allclose(u, 0.9238311052322388, atol=1e-6, rtol=1e-6)   # = C(50,2)/C(52,2)
    assert abs(1225 / 1326 - 0.9238311052322388) < 1e-7


def test_unblocked_delta_and_double_half_delta():
    shared = OC.combo_onehot().astype(np.float64) @ OC.combo_onehot().astype(np.float64).T
    d = np.zeros((1, H), np.float32)
    d[0, 100] = 1.0
    u = OU.calculate_unblocked_mass(d)[0]
    assert u[100] == 0.0
    assert (u[shared[:, 100] < 0.5] == 1.0).all()
    assert (u[shared[:, 100] > 0.5] == 0.0).all()        # every sharer is fully blocked by a delta
    h1, h2 = 50, 200
    while shared[h1, h2] > 0.5:
        h2 += 1
    d = np.zeros((1, H), np.float32)
    d[0, h1] = d[0, h2] = 0.5
    u = OU.calculate_unblocked_mass(d)[0]
    assert u[h1] == 0.5 and u[h2] == 0.5
    assert (u[(shared[:, h1] < 0.5) & (shared[:, h2] < 0.5)] == 1.0).all()


def test_unblocked_matches_compatibility_product_and_loops():
    rng = np.random.default_rng(0)
    onehot = OC.combo_onehot().astype(np.float64)
    compatible = 1.0 - onehot @ onehot.T + np.eye(H)      # test_card_utils.py:594-600
    compatible[compatible < 0] = 0.0                       # the hand itself shares 2 cards: 1-2+1 = 0
    rows = np.stack([np.full(H, 1.0 / H), rng.dirichlet(np.full(H, 0.3)), rng.random(H) * (rng.random(H) < 0.05)])
    rows = rows.astype(np.float32)
    got = OU.calculate_unblocked_mass(rows)
    np.testing.assert_allclose(got, rows.astype(np.float64) @ compatible, atol=1e-6, rtol=1e-6)
    np.testing.assert_allclose(got[1], OU.unblocked_mass_loops(rows[1]), atol=1e-6, rtol=1e-6)
    np.testing.assert_allclose(OU.unblocked_mass_inclusion_exclusion(rows), got, atol=2e-6, rtol=1e-5)


def test_unblocked_ratio_threshold_and_gather():
    rng = np.random.default_rng(1)
    numer = rng.random((4, H)).astype(np.float32)
    denom = rng.random((2, H)).astype(np.float32)
    denom[1] = 0.0
    r = OU.unblocked_mass_ratio(numer, denom, parent_index=np.array([0, 1, 0, 1]))
    assert (r[1] == 0).all() and (r[3] == 0).all()         # denominator under eps -> 0
    exp = OU.calculate_unblocked_mass(numer[0]) / OU.calculate_unblocked_mass(denom[0])
    np.testing.assert_allclose(r[0], exp, rtol=1e-6)


# ---- showdown -------------------------------------------------------------------------------
def blocked_and_normalised(bel, board):
    """What the evaluator does to the beliefs it is handed (cfr_evaluator.py:766-828): zero the
    board-blocked hands, renormalise.  The showdown formula assumes both."""
    allowed, _ = OC.allowed_hands_for_boards(np.asarray(board, dtype=np.int64)[None])
    bel = bel * allowed[:, None, :]
    return (bel / bel.sum(-1, keepdims=True)).astype(np.float32)


def hrd_for(board):
    board = np.asarray(board, dtype=np.int64)[None]
    allowed, _ = OC.allowed_hands_for_boards(board)
    return OS.init_hand_rank_data(board, allowed)


BOARDS = ["Ac Qh 9d 7s 4h", "Ad Kd Qd Jd 2s", "Ah Kh Qh Jh Th", "7c 7d 7h 2s 2c", "9s 8s 7s 6s 2d"]


@pytest.mark.parametrize("text", BOARDS)
def test_showdown_matches_pair_enumeration(text):
    board = np.array(parse_board(text))
    rng = np.random.default_rng(abs(hash(text)) % 1000)
    hrd = hrd_for(board)
    cases = [blocked_and_normalised(np.full((1, 2, H), 1.0 / H, np.float32), board), random_ranges(rng, board[None], alpha=0.3)]
    sparse = random_ranges(rng, board[None]) * (rng.random((1, 2, H)) < 0.03)
    cases.append((sparse / sparse.sum(-1, keepdims=True)).astype(np.float32))
    for bel in cases:
        pot = np.array([[0.7, 0.45]], np.float32)
        got = OS.showdown_value_both(bel, hrd, pot, np.ones(1, np.float32))
        for hero in (0, 1):
            exp = OS.showdown_value_bruteforce(board, bel[0, 1 - hero], float(pot[0, hero]))
            np.testing.assert_allclose(got[0, hero], exp, atol=3e-6, rtol=1e-5)


def test_showdown_sure_win_sure_loss_and_all_ties():
    # test_rebel_cfr_evaluator.py:1241-1300: hero holds the straight flush on Ad Kd Qd Jd 2s
    board = np.array(parse_board("Ad Kd Qd Jd 2s"))
    suit = parse_board("Ad")[0] // 13
    hero = OC.combo_index(C(7, suit), C(8, suit))          # 9d Td
    bel = np.zeros((1, 2, H), np.float32)
    bel[0, 0, hero] = 1.0
    bel[0, 1] = 1.0 / (H - 1)
    bel[0, 1, hero] = 0.0
    bel = blocked_and_normalised(bel, board)
    hrd = hrd_for(board)
    pot = np.array([[0.3, 0.3]], np.float32)
    v = OS.showdown_value_both(bel, hrd, pot, np.ones(1, np.float32))
    assert v[0, 0, hero] == pytest.approx(0.3, abs=1e-6)
    ok = OC.mask_conflicting(board) & OC.mask_conflicting(np.array([C(7, suit), C(8, suit)]))
    np.testing.assert_allclose(v[0, 1][ok], -0.3, atol=1e-6)    # everyone compatible loses to it
    assert (v[0, 1][~ok] == 0).all()                            # blocked hands: no villain mass left
    # royal flush on board: every showdown ties
    board = np.array(parse_board("Ah Kh Qh Jh Th"))
    bel = random_ranges(np.random.default_rng(2), board[None])
    v = OS.showdown_value_both(bel, hrd_for(board), pot, np.ones(1, np.float32))
    assert np.abs(v).max() < 1e-6


def test_showdown_properties_on_random_boards():
    rng = np.random.default_rng(3)
    boards = random_boards(rng, 6)
    allowed, _ = OC.allowed_hands_for_boards(boards)
    hrd = OS.init_hand_rank_data(boards, allowed)
    bel = random_ranges(rng, boards)
    pot = (rng.random((6, 2)) + 0.1).astype(np.float32)
    scale = np.ones(6, np.float32)
    v = OS.showdown_value_both(bel, hrd, pot, scale)
    assert (np.abs(v) <= pot[:, :, None] + 1e-6).all()
    assert (v[np.broadcast_to(~allowed[:, None, :], v.shape)] == 0).all()
    # potentials and scale enter linearly
    v2 = OS.showdown_value_both(bel, hrd, pot * np.float32(2.0), scale * np.float32(4.0))
    np.testing.assert_allclose(v2, v * 0.5, atol=1e-6, rtol=1e-5)
    # with equal potentials the game is zero-sum over compatible pairs:
    # sum_h b0[h] m1[h] v0[h] + sum_h b1[h] m0[h] v1[h] = 0, m = compatible opposing mass
    one = np.ones((6, 2), np.float32)
    v = OS.showdown_value_both(bel, hrd, one, scale).astype(np.float64)
    m1 = OU.calculate_unblocked_mass(bel[:, 1]).astype(np.float64)
    m0 = OU.calculate_unblocked_mass(bel[:, 0]).astype(np.float64)
    total = (bel[:, 0] * m1 * v[:, 0]).sum(-1) + (bel[:, 1] * m0 * v[:, 1]).sum(-1)
    assert np.abs(total).max() < 2e-6
