"""GPU parity of the 7-card ranker: bit-exact against the oracle and the golden vectors
written by the reference's own rules.py; called through the reference-named wrappers."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import ranker as R
from oracle import ranker_c as RC

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def K():
    from poker2_amd import rules_hip
    assert rules_hip.triton_is_available(), "libp2hip.so / GPU missing"
    return rules_hip


def seeded_hands(n: int, seed: int = 7) -> np.ndarray:
    rng = np.random.default_rng(seed)
    # argsort of random keys = a uniform shuffle per row; first 7 = 7 distinct cards
    return np.argsort(rng.random((n, 52)), axis=1)[:, :7].astype(np.int8)


def test_golden_vectors_all_dtypes(K, golden_dir):
    g = np.load(os.path.join(golden_dir, "ranker_golden.npz"))
    cards = g["cards"]
    full = (cards >= 0).all(axis=1)
    c7 = cards[full]
    for dt in (torch.int8, torch.int16, torch.int32, torch.int64):
        out = K.rank_7_cards_single_batch_triton(torch.from_numpy(c7.astype(np.int64)).to(dt).cuda())
        assert out.dtype == torch.int32
        assert np.array_equal(out.cpu().numpy(), g["packed"][full]), dt
    planes = torch.from_numpy(R.cards_to_planes(cards.astype(np.int64))).cuda()
    for ff in (False, True):
        out = K.rank_7_planes(planes, flush_first=ff)
        assert np.array_equal(out.cpu().numpy(), g["packed"])  # includes the short hands
    ab = torch.stack([planes[:-1], planes[1:]], dim=1)
    for fn in (K.compare_7_single_batch, K.compare_7_single_batch_triton):
        assert np.array_equal(fn(ab).cpu().numpy(), g["cmp_adjacent"].astype(np.int32))
    assert np.array_equal(K.compare_7_batches(planes[:-1], planes[1:]).cpu().numpy(), g["cmp_adjacent"])
    assert np.array_equal(K.compare_7_batches_triton(planes[:-1], planes[1:]).cpu().numpy(), g["cmp_adjacent"])


def test_reference_test_pairs(K, golden_dir):
    with open(os.path.join(golden_dir, "rules_pairs.json")) as f:
        pairs = json.load(f)["pairs"]
    a = np.array([p["a"] for p in pairs if len(p["a"]) == 7 and len(p["b"]) == 7])
    b = np.array([p["b"] for p in pairs if len(p["a"]) == 7 and len(p["b"]) == 7])
    e = np.array([p["expected"] for p in pairs if len(p["a"]) == 7 and len(p["b"]) == 7], dtype=np.int32)
    cards = torch.from_numpy(np.stack([a, b], axis=1)).to(torch.int16).cuda()
    assert np.array_equal(K.compare_7_cards_single_batch_triton(cards).cpu().numpy(), e)


@pytest.mark.parametrize("n", [1, 255, 256, 257, 1000003])
def test_random_hands_bit_exact(K, n):
    cards = seeded_hands(n, seed=7 + n)
    exp = RC.rank_cards(cards)
    out = K.rank_7_cards_single_batch_triton(torch.from_numpy(cards).cuda())
    assert np.array_equal(out.cpu().numpy(), exp)


def test_config1_full_size(K):
    """2^20 hands of 7 distinct cards, int8 ids, int32 packed rank, bit-exact."""
    cards = seeded_hands(1 << 20, seed=7)
    exp = RC.rank_cards(cards)
    out = K.rank_7_cards_single_batch_triton(torch.from_numpy(cards).cuda())
    assert np.array_equal(out.cpu().numpy(), exp)
    # a permutation of the seven cards never changes the score
    perm = np.random.default_rng(1).permutation(7)
    out2 = K.rank_7_cards_single_batch_triton(torch.from_numpy(np.ascontiguousarray(cards[:, perm])).cuda())
    assert torch.equal(out, out2)


def test_compare_cards_and_duplicates(K):
    rng = np.random.default_rng(3)
    cards = np.stack([seeded_hands(5000, 11), seeded_hands(5000, 12)], axis=1).astype(np.int16)
    cards[::7, 0, 1] = cards[::7, 0, 0]  # a repeated id counts twice towards pairs
    s = RC.rank_cards(cards)
    exp = np.sign(s[:, 0].astype(np.int64) - s[:, 1]).astype(np.int32)
    out = K.compare_7_cards_single_batch_triton(torch.from_numpy(cards).cuda())
    assert np.array_equal(out.cpu().numpy(), exp)
    del rng


def test_input_validation(K):
    with pytest.raises(ValueError):
        K.rank_7_cards_single_batch_triton(torch.zeros(4, 6, dtype=torch.int16, device="cuda"))
    with pytest.raises(ValueError):
        K.rank_7_cards_single_batch_triton(torch.zeros(4, 7, dtype=torch.int16))
    with pytest.raises(ValueError):
        K.compare_7_single_batch_triton(torch.zeros(4, 2, 4, 12, dtype=torch.bool, device="cuda"))
    with pytest.raises(ValueError):
        K.rank_hands_triton(torch.zeros(4, 4, dtype=torch.long, device="cuda"))
    assert K.rank_7_cards_single_batch_triton(torch.zeros(0, 7, dtype=torch.int8, device="cuda")).shape == (0,)


def test_rank_hands_golden_and_oracle(K, golden_dir):
    g = np.load(os.path.join(golden_dir, "ranker_golden.npz"))
    boards = torch.from_numpy(g["boards"].astype(np.int64)).cuda()
    ranks, order = K.rank_hands(boards)
    assert ranks.dtype == torch.int32 and order.dtype == torch.int64
    assert np.array_equal(ranks.cpu().numpy(), g["board_ranks"].astype(np.int32))
    assert np.array_equal(order.cpu().numpy(), g["board_order"].astype(np.int64))
    rng = np.random.default_rng(5)
    b = np.stack([rng.permutation(52)[:5] for _ in range(300)]).astype(np.int64)
    er, eo = R.rank_hands(b)
    ranks, order = K.rank_hands(torch.from_numpy(b).cuda())
    assert np.array_equal(ranks.cpu().numpy(), er) and np.array_equal(order.cpu().numpy(), eo)
    # card-id variant: packed scores + stable argsort, for every board dtype
    ep, eo2 = R.rank_hands_cards(b)
    for dt in (torch.int8, torch.int16, torch.int32, torch.int64):
        p, o = K.rank_hands_triton(torch.from_numpy(b).to(dt).cuda())
        assert np.array_equal(p.cpu().numpy(), ep) and np.array_equal(o.cpu().numpy(), eo2)


def test_comparison_vector_and_scalar_compare(K, golden_dir):
    """create_comparison_vector / compare_7 / HandType of src/p2/env/rules.py against the fields
    the reference itself produced for the golden hands."""
    g = np.load(str(golden_dir) + "/ranker_golden.npz")
    cards, fields = g["cards"].astype(np.int64), g["fields"].astype(np.int32)
    n = 1024
    planes = np.zeros((n, 1, 4, 13), dtype=bool)
    for i in range(n):
        planes[i, 0, cards[i] // 13, cards[i] % 13] = True
    got = K.create_comparison_vector(torch.from_numpy(planes).cuda()).cpu().numpy()
    assert got.shape == (n, 1, 6) and np.array_equal(got[:, 0], fields[:n])
    assert {int(x) for x in np.unique(got[:, 0, 0])} <= {t.value for t in K.HandType}
    for i in range(0, 40, 2):
        exp = int(np.sign(int(g["packed"][i]) - int(g["packed"][i + 1])))
        assert K.compare_7(cards[i].tolist(), cards[i + 1].tolist()) == exp
    from poker2_amd import fused_cfr_hip as F
    from poker2_amd.evaluator import GraphedCFRIteration
    assert F.GraphedCFRIteration is GraphedCFRIteration
    stats = F.ParentBeliefUnblockedStats(torch.rand(5, 2, 1326, device="cuda"))
    t, s, cs = stats.slice_for_player(torch.tensor([0, 1, 1, 0, 1], device="cuda"))
    assert t.shape == (5, 1326) and s.shape == (5,) and cs.shape == (5, 52)
    torch.testing.assert_close(cs.sum(-1), 2 * s, rtol=1e-5, atol=1e-5)


def test_repeated_card_ids_score_like_the_reference_kernel(K, golden_dir):
    """Hands that repeat a card id, scored by the reference's own card-id kernel run under Triton's CPU
    interpreter (tests/golden/gen_ranker_cards_golden.py): the repeat counts again towards pairs / trips /
    quads and carries into the next bit of its suit's mask (rules_triton.py:421-440).  Every input dtype,
    the comparison entry point, and ``rank_hands_triton`` on three boards — where every combo that holds a
    board card is such a hand — bit for bit."""
    g = np.load(os.path.join(golden_dir, "ranker_cards_golden.npz"))
    hands, scores = g["hands"], g["scores"]
    assert int((np.sort(hands, axis=1)[:, 1:] == np.sort(hands, axis=1)[:, :-1]).any(axis=1).sum()) >= 300
    for dt in (torch.int8, torch.int16, torch.int32, torch.int64):
        out = K.rank_7_cards_single_batch_triton(torch.from_numpy(hands.astype(np.int64)).to(dt).cuda())
        assert np.array_equal(out.cpu().numpy(), scores), dt
    pairs = np.stack([hands[:-1], hands[1:]], axis=1).astype(np.int16)
    exp = np.sign(scores[:-1].astype(np.int64) - scores[1:]).astype(np.int32)
    assert np.array_equal(K.compare_7_cards_single_batch_triton(torch.from_numpy(pairs).cuda()).cpu().numpy(), exp)
    for dt in (torch.int8, torch.int64):
        p, o = K.rank_hands_triton(torch.from_numpy(g["boards"]).to(dt).cuda())
        assert np.array_equal(p.cpu().numpy(), g["hand_ranks"]) and np.array_equal(o.cpu().numpy(), g["sorted_indices"])
