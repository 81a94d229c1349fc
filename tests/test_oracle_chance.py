"""CPU: pins the oracle's restatement of the single-card chance node
(src/p2/search/chance_node_helper.py:360-479)."""
import numpy as np

from oracle import cards as OC
from oracle import chance as OCH
from tests.helpers import random_boards

H = 1326


def setup(rng, b, k):
    boards = np.full((b, 5), -1, dtype=np.int64)
    boards[:, :k] = random_boards(rng, b, k)
    pre = rng.gamma(0.5, size=(b, 2, H)).astype(np.float32)
    pre /= pre.sum(-1, keepdims=True)
    return boards, pre


def test_expand_against_per_sample_loop():
    rng = np.random.default_rng(0)
    boards, pre = setup(rng, 3, 4)
    pre[1, 0] = 0.0                         # a dead range: every sample of it falls back to uniform
    pre[2, 1, :] = 0.0
    pre[2, 1, OC.combo_index(0, 1)] = 1.0   # a delta range: dead only on samples that deal card 0 or 1
    post, board_samples, root_lookup = OCH.expand(pre, boards)
    cm = OC.hand_combos()
    s = 0
    for i in range(3):
        for c in range(52):
            if c in boards[i]:
                continue
            assert root_lookup[s] == i
            assert list(board_samples[s]) == list(boards[i, :4]) + [c]
            dead = set(boards[i, :4].tolist()) | {c}
            ok = np.array([cm[h, 0] not in dead and cm[h, 1] not in dead for h in range(H)])
            assert ok.sum() == 47 * 46 // 2
            for p in range(2):
                x = np.where(ok, pre[i, p].astype(np.float64), 0.0)
                exp = x / x.sum() if x.sum() > 1e-12 else ok / ok.sum()
                np.testing.assert_allclose(post[s, p], exp, rtol=2e-6, atol=1e-9)
            s += 1
    assert s == post.shape[0] == 3 * 48


def test_sample_counts_and_order_for_mixed_streets():
    rng = np.random.default_rng(1)
    boards = np.full((4, 5), -1, dtype=np.int64)
    boards[0, :3] = [5, 17, 40]
    boards[1, :4] = [0, 1, 2, 3]
    boards[2, :3] = [51, 50, 49]
    pre = rng.random((4, 2, H)).astype(np.float32)
    post, board_samples, root_lookup = OCH.expand(pre, boards)
    assert np.bincount(root_lookup).tolist() == [49, 48, 49, 52]
    assert (np.diff(root_lookup) >= 0).all()
    for i, k in enumerate([3, 4, 3, 0]):
        dealt = board_samples[root_lookup == i][:, k]
        assert (np.diff(dealt) > 0).all() and not set(dealt) & set(boards[i])
    np.testing.assert_allclose(post.sum(-1), 1.0, atol=1e-5)


def test_closed_forms_echo_and_board_models():
    rng = np.random.default_rng(2)
    boards, pre = setup(rng, 5, 4)
    roots = np.array([4, 0, 2])
    ctx = np.zeros((5, 1), np.float32)
    zeros = np.zeros(5, np.int64)

    def echo(context, street, to_act, board, beliefs):
        return beliefs.reshape(-1, 2, H)
    got = OCH.single_card_chance_values(roots, ctx, zeros, zeros, pre, boards, echo)
    onehot = OC.combo_onehot()
    for j, r in enumerate(roots):
        acc = np.zeros((2, H))
        for c in range(52):
            if c in boards[r]:
                continue
            dead = np.zeros(52, bool)
            dead[boards[r, :4]] = True
            dead[c] = True
            ok = ~(onehot & dead[None, :]).any(axis=1)
            x = pre[r].astype(np.float64) * ok
            acc += x / x.sum(-1, keepdims=True)
        np.testing.assert_allclose(got[j], acc / 48, rtol=1e-5, atol=1e-8)
    # ranges sum to one, so does their mean; a hand that holds a dealt card contributes 0 there
    np.testing.assert_allclose(got.sum(-1), 1.0, atol=1e-5)

    def board_rank_sum(context, street, to_act, board, beliefs):
        v = (np.where(board >= 0, board % 13, 0).sum(axis=1) % H).astype(np.float32)
        return np.broadcast_to(v[:, None, None], (board.shape[0], 2, H))
    got = OCH.single_card_chance_values(roots, ctx, zeros, zeros, pre, boards, board_rank_sum)
    for j, r in enumerate(roots):
        base = (boards[r, :4] % 13).sum()
        exp = np.mean([(base + c % 13) % H for c in range(52) if c not in boards[r]])
        np.testing.assert_allclose(got[j], exp, rtol=1e-6)


def test_empty_input_and_shapes():
    out = OCH.single_card_chance_values(np.zeros(0, np.int64), np.zeros((0, 1)), np.zeros(0), np.zeros(0),
                                        np.zeros((0, 2, H), np.float32), np.zeros((0, 5), np.int64), None)
    assert out.shape == (0, 2, H)
    rng = np.random.default_rng(3)
    boards, pre = setup(rng, 4, 4)
    out = OCH.single_card_chance_values(np.arange(4), np.zeros((4, 1)), np.zeros(4), np.zeros(4), pre, boards,
                                        lambda c, s, t, b, x: np.zeros((b.shape[0], 2, H), np.float32))
    assert out.shape == (4, 2, H) and out.dtype == np.float32 and not out.any()


def test_oracle_matches_vectors_from_the_reference_helper(golden_dir):
    """tests/golden/chance_golden.npz: outputs of the reference's own single_card_chance_values
    (run by tests/golden/gen_chance_golden.py) for an echo network and a board-and-range network,
    mixed turn / flop boards, a dead range and a delta range."""
    g = np.load(str(golden_dir) + "/chance_golden.npz")
    board, pre, roots = g["board"], g["pre_beliefs"], g["root_indices"]
    n = board.shape[0]

    def echo(context, street, to_act, b, beliefs):
        return beliefs.reshape(-1, 2, H)

    def board_and_range(context, street, to_act, b, beliefs):
        w = 1.0 + np.where(b >= 0, b % 13, 0).sum(axis=1).astype(np.float32) / np.float32(100.0)
        return beliefs.reshape(-1, 2, H) * w[:, None, None]
    for name, fn in (("echo", echo), ("board_and_range", board_and_range)):
        got = OCH.single_card_chance_values(roots, np.zeros((n, 1), np.float32), np.full(n, 3), np.zeros(n, np.int64),
                                            pre, board, fn)
        np.testing.assert_allclose(got, g[name], rtol=1e-5, atol=1e-8)


# ---- three-card (flop) chance node (src/p2/search/chance_node_helper.py:76-357) ------------

def flop_models():
    """numpy twins of the networks in tests/golden/gen_flop_chance_golden.py."""
    def echo(context, street, to_act, board, beliefs):
        return beliefs.reshape(-1, 2, H).astype(np.float32)

    def suit_aware(context, street, to_act, board, beliefs):
        b = beliefs.reshape(-1, 2, H).astype(np.float32)
        w = (1.0 + (board[:, 0] // 13).astype(np.float32) / np.float32(10.0)
             + (board[:, 2] % 13).astype(np.float32) / np.float32(100.0)).astype(np.float32)
        h = (np.arange(H) % 7).astype(np.float32) * np.float32(0.001)
        return b * w[:, None, None] + h[None, None, :] * np.array([1.0, 2.0], dtype=np.float32)[None, :, None]

    return {"echo": echo, "suit_aware": suit_aware}


def test_canonical_flops_and_suit_maps_match_the_reference_cache(golden_dir):
    g = np.load(str(golden_dir) + "/flop_chance_golden.npz")
    canonical, count, flop_to_class = OCH.canonical_flops()
    assert np.array_equal(canonical, g["flop_id_to_canonical"].astype(np.int64))
    assert np.array_equal(count, g["flop_id_to_count"].astype(np.int64))
    assert np.array_equal(flop_to_class, g["flop_to_canon"].astype(np.int64))
    assert np.array_equal(OCH.suit_permutations(), g["suit_permutations"].astype(np.int64))
    perms = OCH.combo_suit_perms()
    assert np.array_equal(perms, g["combo_perm"].astype(np.int64))
    assert np.array_equal(np.argsort(perms, axis=1), g["combo_perm_inverse"].astype(np.int64))
    # what the mathematics fixes: 1755 classes; sizes by rank pattern are 4 (trips), 12 or 24 ... and sum to C(52,3)
    assert canonical.shape == (1755, 3) and count.sum() == 22100
    ranks = canonical % 13
    trips = (ranks[:, 0] == ranks[:, 1]) & (ranks[:, 1] == ranks[:, 2])
    assert trips.sum() == 13 and (count[trips] == 4).all()
    distinct = (ranks[:, 0] != ranks[:, 1]) & (ranks[:, 1] != ranks[:, 2])
    # three distinct ranks: monotone (4), two-tone (3 x 12), rainbow (24) per rank triple
    assert distinct.sum() == 286 * 5 and sorted(set(count[distinct].tolist())) == [4, 12, 24]
    assert (~trips & ~distinct).sum() == 13 * 12 * 2 and set(count[~trips & ~distinct].tolist()) == {12}
    # every row of the hand map is a permutation, the identity comes first
    assert (np.sort(perms, axis=1) == np.arange(H)).all() and (perms[0] == np.arange(H)).all()


def test_flop_oracle_matches_vectors_from_the_reference_helper(golden_dir):
    g = np.load(str(golden_dir) + "/flop_chance_golden.npz")
    canonical, count, _ = OCH.canonical_flops()
    perms = OCH.combo_suit_perms()
    pre, roots = g["pre_beliefs"], g["root_indices"]
    n = pre.shape[0]
    ctx, st, ta = np.zeros((n, 1), np.float32), np.zeros(n, np.int64), np.zeros(n, np.int64)
    for name, fn in flop_models().items():
        cases = {"all": dict(), "all_perm6": dict(perm_rows=list(g["all_perm6_rows"])),
                 "sample256_perm6": dict(sample_idx=g["sample256_idx"].astype(np.int64),
                                         perm_rows=list(g["sample256_rows"]))}
        for mode, kw in cases.items():
            got = OCH.flop_chance_values(roots, ctx, st, ta, pre, fn, canonical, count, perms, **kw)
            ref = g[f"{name}_{mode}"]
            np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-7, err_msg=f"{name} {mode}")


def test_flop_closed_form_suit_equivariant_network():
    """A network whose answer moves with the suits (here: echo of ranges that are themselves
    suit-symmetric, i.e. uniform) gives, through classes x orbit mean, exactly the plain mean over
    all 22100 flops of the expanded range: every hand is blocked by C(52,3) - C(50,3) flops."""
    canonical, count, _ = OCH.canonical_flops()
    perms = OCH.combo_suit_perms()
    pre = np.full((1, 2, H), 1.0 / H, dtype=np.float32)
    got = OCH.flop_chance_values(np.array([0]), np.zeros((1, 1)), np.zeros(1, np.int64), np.zeros(1, np.int64), pre,
                                 flop_models()["echo"], canonical, count, perms)
    expected = (19600.0 / 22100.0) / 1176.0
    np.testing.assert_allclose(got, expected, rtol=1e-5)


def test_flop_expand_against_per_flop_loop():
    rng = np.random.default_rng(3)
    pre = rng.gamma(0.5, size=(2, 2, H)).astype(np.float32)
    pre /= pre.sum(-1, keepdims=True)
    pre[1, 0] = 0.0
    flops = np.array([[0, 13, 26], [51, 3, 20], [12, 11, 10]], dtype=np.int64)
    post = OCH.flop_expand(pre, flops)
    cm = OC.hand_combos()
    for k, f in enumerate(flops):
        ok = np.array([cm[h, 0] not in f and cm[h, 1] not in f for h in range(H)])
        assert ok.sum() == 1176
        for i in range(2):
            for p in range(2):
                x = np.where(ok, pre[i, p].astype(np.float64), 0.0)
                exp = x / x.sum() if x.sum() > 1e-12 else ok / ok.sum()
                np.testing.assert_allclose(post[i, k, p], exp, rtol=1e-5, atol=1e-9)
