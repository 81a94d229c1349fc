"""GPU parity of the river showdown evaluator against the oracle (cumsum restatement and
brute force) on the boards the reference's tests use and on seeded random boards."""
import numpy as np
import pytest
import torch

from oracle import cards as OC
from oracle import showdown as OS
from tests.helpers import H, C, random_boards, random_ranges

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 2e-6


@pytest.fixture(scope="module")
def K():
    from poker2_amd import rules_hip
    assert rules_hip.triton_is_available(), "libp2hip.so / GPU missing"
    return rules_hip


def run_hip(K, boards, beliefs, potential, scale, triton_order=True):
    tables = K.build_showdown_tables(torch.from_numpy(boards).cuda(), triton_order=triton_order)
    out = K.showdown_value_both(torch.from_numpy(beliefs).cuda(), tables,
                                torch.from_numpy(potential).cuda(), torch.from_numpy(scale).cuda())
    return out.cpu().numpy()


def oracle_both(boards, beliefs, potential, scale):
    allowed, _ = OC.allowed_hands_for_boards(boards)
    hrd = OS.init_hand_rank_data(boards, allowed)
    return OS.showdown_value_both(beliefs, hrd, potential, scale)


NAMED_BOARDS = np.array([
    [C(12, 3), C(10, 1), C(7, 2), C(5, 0), C(2, 1)],    # Ac Qh 9d 7s 4h
    [C(12, 2), C(11, 2), C(10, 2), C(9, 2), C(0, 0)],   # Ad Kd Qd Jd 2s
    [C(12, 1), C(11, 1), C(10, 1), C(9, 1), C(8, 1)],   # Ah Kh Qh Jh Th (everything ties)
    [C(12, 0), C(9, 1), C(5, 3), C(3, 0), C(0, 2)],     # As Jh 7c 5s 2d
    [C(8, 3), C(8, 1), C(8, 0), C(5, 2), C(5, 1)],      # Tc Th Ts 7d 7h
    [C(5, 2), C(4, 2), C(3, 2), C(2, 2), C(1, 2)],      # 7d 6d 5d 4d 3d
    [C(12, 3), C(11, 2), C(10, 1), C(9, 0), C(7, 3)],   # Ac Kd Qh Js 9c
], dtype=np.int64)


@pytest.mark.parametrize("triton_order", [True, False])
def test_named_boards_vs_oracle_and_bruteforce(K, triton_order):
    rng = np.random.default_rng(42)
    boards = NAMED_BOARDS
    m = boards.shape[0]
    bel = random_ranges(rng, boards)
    pot = np.tile(np.array([[200.0, 200.0]], dtype=np.float32), (m, 1))
    scale = np.full(m, 1000.0, dtype=np.float32)
    out = run_hip(K, boards, bel, pot, scale, triton_order)
    exp = oracle_both(boards, bel, pot, scale)
    np.testing.assert_allclose(out, exp, rtol=RTOL, atol=ATOL)
    for i in range(m):
        for hero in (0, 1):
            bf = OS.showdown_value_bruteforce(boards[i], bel[i, 1 - hero], 0.2)
            np.testing.assert_allclose(out[i, hero], bf, rtol=1e-4, atol=3e-6)
    assert np.abs(out[2]).max() == 0.0  # royal flush on board: all ties


def test_uniform_and_delta_ranges(K):
    boards = NAMED_BOARDS[[0, 1]]
    allowed, prob = OC.allowed_hands_for_boards(boards)
    bel = np.stack([prob, prob], axis=1).astype(np.float32)
    pot = np.array([[150.0, 250.0], [90.0, 90.0]], dtype=np.float32)
    scale = np.array([1000.0, 450.0], dtype=np.float32)
    out = run_hip(K, boards, bel, pot, scale)
    np.testing.assert_allclose(out, oracle_both(boards, bel, pot, scale), rtol=RTOL, atol=ATOL)
    assert np.all(out[:, 0][~allowed] == 0) and np.all(out[:, 1][~allowed] == 0)
    assert np.abs(out[0, 0]).max() <= 0.15 + 1e-6 and np.abs(out[0, 1]).max() <= 0.25 + 1e-6
    # villain holds one known hand (T9 of the board's suit = straight flush on board 1)
    hero = OC.combo_index(C(8, 2), C(7, 2))
    bel2 = bel.copy()
    bel2[1, 1] = 0.0
    bel2[1, 1, hero] = 1.0
    out2 = run_hip(K, boards, bel2, pot, scale)
    ok = allowed[1] & OC.mask_conflicting([C(8, 2), C(7, 2)])
    np.testing.assert_allclose(out2[1, 0][ok], -90.0 / 450.0, rtol=1e-6)
    assert np.all(out2[1, 0][~ok] == 0)
    np.testing.assert_allclose(out2, oracle_both(boards, bel2, pot, scale), rtol=RTOL, atol=ATOL)


def test_config2_shape_properties(K):
    """B=4096 boards, Dirichlet(0.5) ranges, pot 1.0: compare a slice with the oracle and
    check size-independent properties on all of it."""
    rng = np.random.default_rng(42)
    b = 4096
    boards = random_boards(rng, b)
    bel = random_ranges(rng, boards)
    pot = np.ones((b, 2), dtype=np.float32)
    scale = np.ones(b, dtype=np.float32)
    out = run_hip(K, boards, bel, pot, scale)
    sl = slice(0, 96)
    np.testing.assert_allclose(out[sl], oracle_both(boards[sl], bel[sl], pot[sl], scale[sl]), rtol=RTOL, atol=ATOL)
    allowed, _ = OC.allowed_hands_for_boards(boards)
    assert np.isfinite(out).all() and np.abs(out).max() <= 1.0 + 1e-5
    assert np.all(out[:, 0][~allowed] == 0) and np.all(out[:, 1][~allowed] == 0)
    # zero-sum: sum_h0 b0[h0] * m1(h0) * EV0[h0] = - sum_h1 b1[h1] * m0(h1) * EV1[h1]
    from oracle.unblocked import calculate_unblocked_mass
    m1 = calculate_unblocked_mass(bel[:256, 1])
    m0 = calculate_unblocked_mass(bel[:256, 0])
    v0 = (bel[:256, 0] * m1 * out[:256, 0]).sum(-1)
    v1 = (bel[:256, 1] * m0 * out[:256, 1]).sum(-1)
    np.testing.assert_allclose(v0, -v1, atol=2e-5)
    # scaling potential scales the result; table_row indirection gives the same answer
    tables = K.build_showdown_tables(torch.from_numpy(boards).cuda())
    idx = torch.arange(b - 1, -1, -1, device="cuda")
    out_rev = K.showdown_value_both(torch.from_numpy(bel).cuda().flip(0).contiguous(), tables,
                                    torch.from_numpy(pot * 3).cuda(), torch.from_numpy(scale).cuda(), table_row=idx)
    np.testing.assert_allclose(out_rev.cpu().numpy()[::-1], out * 3, rtol=1e-6, atol=1e-7)


def test_blocked_mass_in_villain_range(K):
    """Mass on board-blocked combos is tolerated exactly as the reference tolerates it."""
    rng = np.random.default_rng(9)
    boards = random_boards(rng, 8)
    bel = rng.random((8, 2, H)).astype(np.float32)
    bel /= bel.sum(-1, keepdims=True)
    pot = np.full((8, 2), 300.0, dtype=np.float32)
    scale = np.full(8, 900.0, dtype=np.float32)
    # same ranker on both sides: the two rankers order board-blocked combos differently
    np.testing.assert_allclose(run_hip(K, boards, bel, pot, scale, triton_order=False),
                               oracle_both(boards, bel, pot, scale), rtol=RTOL, atol=ATOL)


def test_empty(K):
    tables = K.build_showdown_tables(torch.zeros(0, 5, dtype=torch.long, device="cuda"))
    out = K.showdown_value_both(torch.zeros(0, 2, H, device="cuda"), tables, torch.zeros(0, 2, device="cuda"),
                                torch.zeros(0, device="cuda"))
    assert out.shape == (0, 2, H)


def test_ev_from_strength_sorted_inputs_matches_oracle_and_refuses_bad_rows():
    """``showdown_ev_triton`` (fused_cfr_triton.py:2271-2314): the same EV from inputs that are
    already in strength order; un-sorting, board mask and chips are the caller's."""
    from poker2_amd import fused_cfr_hip as F
    rng = np.random.default_rng(9)
    boards = np.concatenate([NAMED_BOARDS, random_boards(rng, 9)])
    m = boards.shape[0]
    bel = random_ranges(rng, boards)
    allowed, _ = OC.allowed_hands_for_boards(boards)
    hrd = OS.init_hand_rank_data(boards, allowed)
    ones = np.ones((m, 2), np.float32)
    exp = OS.showdown_value(bel, 0, hrd, ones, ones[:, 0])                   # hero 0, potential = scale = 1
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()       # noqa: E731
    order, inv = dev(hrd.sorted_indices), dev(hrd.inv_sorted)
    c1, c2 = dev(hrd.hands_c1c2_sorted[..., 0]), dev(hrd.hands_c1c2_sorted[..., 1])          # int64, as the reference keeps them
    b_sorted = torch.gather(dev(bel[:, 1]), 1, order).contiguous()
    ev_sorted = F.showdown_ev_triton(b_sorted, c1, c2, dev(hrd.L_idx), dev(hrd.R_idx))
    got = (torch.gather(ev_sorted, 1, inv) * dev(allowed).float()).cpu().numpy()
    np.testing.assert_allclose(got, exp, rtol=RTOL, atol=ATOL)
    # the two cards of a hand may come in either order
    ev_swapped = F.showdown_ev_triton(b_sorted, c2, c1, dev(hrd.L_idx), dev(hrd.R_idx))
    assert torch.equal(ev_swapped, ev_sorted)
    assert F.showdown_ev_triton(b_sorted[:0].contiguous(), c1[:0], c2[:0], dev(hrd.L_idx)[:0], dev(hrd.R_idx)[:0]).shape == (0, H)
    # rows that are no permutation of the 1326 hands, or whose tie groups do not hold their position
    twice = c1.clone()
    twice[3, 10], c2_twice = c1[3, 11], c2.clone()
    c2_twice[3, 10] = c2[3, 11]
    with pytest.raises(ValueError):
        F.showdown_ev_triton(b_sorted, twice, c2_twice, dev(hrd.L_idx), dev(hrd.R_idx))
    off = c1.clone()
    off[0, 0] = 52
    with pytest.raises(ValueError):
        F.showdown_ev_triton(b_sorted, off, c2, dev(hrd.L_idx), dev(hrd.R_idx))
    late = dev(hrd.L_idx).clone()
    late[2, 100] = 101
    with pytest.raises(ValueError):
        F.showdown_ev_triton(b_sorted, c1, c2, late, dev(hrd.R_idx))
    with pytest.raises(NotImplementedError):
        F.showdown_ev_triton(b_sorted, c1, c2, dev(hrd.L_idx), dev(hrd.R_idx), eps=1e-6)
    torch.cuda.synchronize()


# --- the remaining scenarios of the reference's showdown tests (tests/test_rebel_cfr_evaluator.py:1327-1472),
# restated as data: board "Ac Kd Qh Js 9c", chips 100 each in a pot of 200 over a scale of 1000
BROADWAY_BOARD = NAMED_BOARDS[6:7]


def _scenario(K, villain_range):
    from oracle import ranker as ORK
    boards = BROADWAY_BOARD
    allowed, prob = OC.allowed_hands_for_boards(boards)
    bel = np.stack([prob, prob], axis=1).astype(np.float32)
    bel[0, 1] = villain_range
    pot = np.array([[100.0, 100.0]], dtype=np.float32)
    scale = np.array([1000.0], dtype=np.float32)
    out = run_hip(K, boards, bel, pot, scale)
    np.testing.assert_allclose(out, oracle_both(boards, bel, pot, scale), rtol=RTOL, atol=ATOL)
    combos = OC.hand_combos()
    cards7 = np.concatenate([np.tile(boards[0], (H, 1)), combos], axis=1)
    strength = ORK.rank_cards(cards7)          # board-blocked hands repeat a card; they are masked below
    return out[0], strength, allowed[0]


@pytest.mark.parametrize("villain", [(C(12, 0), C(11, 1)), (C(10, 2), C(9, 3)), (C(8, 0), C(7, 0)), (C(6, 1), C(5, 1))])
def test_villain_holds_one_known_hand(K, villain):
    """:1376-1437 — every compatible hero hand that beats the villain's wins the whole potential, every weaker
    one loses it, equal ones and the villain's own hand get nothing."""
    v = OC.combo_index(*villain)
    rng = np.zeros(H, dtype=np.float32)
    rng[v] = 1.0
    ev, strength, allowed = _scenario(K, rng)
    ok = allowed & OC.mask_conflicting(list(villain))
    better, worse, ties = ok & (strength > strength[v]), ok & (strength < strength[v]), ok & (strength == strength[v])
    assert better.any() or worse.any()
    np.testing.assert_allclose(ev[0][better], 0.1, rtol=1e-6)
    np.testing.assert_allclose(ev[0][worse], -0.1, rtol=1e-6)
    assert np.all(ev[0][ties] == 0) and ev[0][v] == 0 and np.all(ev[0][~ok] == 0)


def test_villain_holds_one_of_two_hands(K):
    """:1440-1472 — half the mass on As Kh (aces and kings), half on Qd Jc (queens and jacks): a hand that beats
    both wins the potential, one between them breaks even, one below both loses it."""
    h1, h2 = OC.combo_index(C(12, 0), C(11, 1)), OC.combo_index(C(10, 2), C(9, 3))
    rng = np.zeros(H, dtype=np.float32)
    rng[h1] = rng[h2] = 0.5
    ev, strength, allowed = _scenario(K, rng)
    winner = OC.combo_index(C(8, 0), C(0, 1))      # Ts 2h: the ten completes the broadway straight
    splitter = OC.combo_index(C(11, 0), C(10, 3))  # Ks Qc: beats QJ, loses to AK
    loser = OC.combo_index(C(2, 0), C(0, 2))       # 4s 2d: loses to both
    assert strength[winner] > max(strength[h1], strength[h2])
    assert strength[h2] < strength[splitter] < strength[h1]
    assert strength[loser] < min(strength[h1], strength[h2])
    np.testing.assert_allclose(ev[0][[winner, splitter, loser]], [0.1, 0.0, -0.1], rtol=1e-6, atol=1e-9)


def test_evaluator_answers_per_player_like_the_reference(K):
    """`_showdown_value(beliefs, hero)` (cfr_evaluator.py:492) is the hero's half of `_showdown_value_both`."""
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.tree import RootStates
    rng = np.random.default_rng(5)
    boards = NAMED_BOARDS[[0, 3, 6]]
    bel = random_ranges(rng, boards)
    roots = RootStates.at_round_start(3, np.full(3, 200), np.tile([[800, 800]], (3, 1)), boards)
    ev = HipSparseCFREvaluator(None, torch.device("cuda"), river_dcfr_config(3, iterations=2, depth=2))
    ev.initialize_subgame(roots, np.arange(3), torch.from_numpy(bel))
    ev.prepare_search()
    b = ev.beliefs[ev.showdown_indices]
    both = ev._showdown_value_both(b)
    assert both.shape == (ev.showdown_indices.numel(), 2, H) and float(both.abs().max()) > 0
    for hero in (0, 1):
        assert torch.equal(ev._showdown_value(b, hero), both[:, hero])
