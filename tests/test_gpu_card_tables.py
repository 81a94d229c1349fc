"""GPU twin of tests/test_card_tables.py: the DEVICE copy of the combo table (csrc/common.h
``p2_combo`` and ``p2_combo_index``) read back through kernels that index with it, and the
evaluator's per-node board masks, all bit-exact."""
import numpy as np
import pytest
import torch

from oracle import cards as OC
from tests.helpers import random_boards, random_ranges

pytestmark = pytest.mark.gpu
H = 1326


def test_device_combo_table_through_unblocked_mass_of_delta_ranges():
    """out[g] = S - cs[a_g] - cs[b_g] + t[g] for the delta range at hand h is 1 where g shares no
    card with h and 0 elsewhere (h itself: 1 - 1 - 1 + 1): the 1326 rows are the compatibility
    table, computed from the device table's cards and its closed-form index."""
    from poker2_amd.card_utils import calculate_unblocked_mass, combo_compatible_tensor
    out = calculate_unblocked_mass(torch.eye(H, device="cuda"))
    assert torch.equal(out, combo_compatible_tensor().float().cuda())
    assert np.array_equal(out.cpu().numpy() > 0.5, OC.combo_compatible())


def test_device_combo_table_through_the_ranker():
    """rank_hands_triton scores combo h from the device table's cards (a[h], b[h]); the card-id
    ranker fed with the HOST table's cards must give the same 1326 scores, and the returned order
    must be the stable argsort of them."""
    from poker2_amd import rules_hip
    from poker2_amd.card_utils import hand_combos_tensor
    rng = np.random.default_rng(12)
    boards = torch.from_numpy(random_boards(rng, 6)).cuda()
    scores, order = rules_hip.rank_hands_triton(boards)
    combos = hand_combos_tensor().cuda()
    seven = torch.cat([combos[None].expand(6, -1, -1), boards[:, None, :].expand(-1, H, -1)], dim=2)
    direct = rules_hip.rank_7_cards_single_batch_triton(seven.reshape(-1, 7).to(torch.int16)).reshape(6, H)
    assert torch.equal(scores, direct)
    assert torch.equal(order, torch.argsort(scores, dim=1, stable=True))


def test_device_combo_table_through_the_chance_expansion_mask():
    """The expansion zeroes exactly the hands that hold the dealt card or a board card: the masks
    of all samples against the host one-hot table."""
    from poker2_amd import chance_node_helper as K
    rng = np.random.default_rng(13)
    boards = np.full((4, 5), -1, dtype=np.int64)
    boards[:, :4] = random_boards(rng, 4, 4)
    boards[3, 3] = -1
    pre = torch.full((4, 2, H), 1.0 / H, device="cuda")
    post, board_samples, _, _ = K.chance_expand(pre, torch.arange(4).cuda(), torch.from_numpy(boards).cuda())
    oh = OC.combo_onehot()
    bs = board_samples.cpu().numpy()
    expect = np.stack([~oh[:, row[row >= 0]].any(axis=1) for row in bs])
    got = post.cpu().numpy() > 0
    assert np.array_equal(got[:, 0], expect) and np.array_equal(got[:, 1], expect)


@pytest.mark.parametrize("street,cards", [(1, 3), (2, 4), (3, 5)])
def test_evaluator_board_masks_on_flop_turn_river(street, cards):
    """allowed_hands / allowed_hands_prob of every node (cfr_evaluator.py:811-819): the root's
    board mask fanned out over its subtree, C(52-k, 2) hands allowed, uniform over them."""
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.tree import RootStates
    rng = np.random.default_rng(20 + street)
    n = 5
    boards = random_boards(rng, n)
    boards[:, cards:] = -1
    beliefs = random_ranges(rng, boards)
    roots = RootStates.at_round_start(street, np.full(n, 200), np.tile([[800, 800]], (n, 1)), boards,
                                      button=np.arange(n) % 2)
    ev = HipSparseCFREvaluator(None, torch.device("cuda"), river_dcfr_config(n, iterations=2, depth=2))
    ev.initialize_subgame(roots, np.arange(n), torch.from_numpy(beliefs))
    allowed, prob = OC.allowed_hands_for_boards(boards)
    root_of = ev.tree.root_index
    assert ev.allowed_hands.dtype == torch.bool and ev.allowed_hands.shape == (ev.total_nodes, H)
    assert np.array_equal(ev.allowed_hands.cpu().numpy(), allowed[root_of])
    assert np.array_equal(ev.allowed_hands_prob.cpu().numpy(), prob[root_of])
    count = (52 - cards) * (51 - cards) // 2
    assert (ev.allowed_hands.sum(dim=1) == count).all()
    assert np.array_equal(np.unique(ev.allowed_hands_prob.cpu().numpy()), np.array([0.0, np.float32(1.0) / np.float32(count)], dtype=np.float32))
