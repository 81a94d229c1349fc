"""GPU parity of the chance nodes (single card: expansion + mean kernels; flop: expansion +
suit-orbit mean kernels; the ChanceNodeHelper mirror) against the oracle and the vectors written
by the reference's own helper, on the cases of the reference's
tests/test_chance_node_helper.py:426-590 and on seeded mixed-street inputs."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import chance as OCH
from tests.helpers import random_boards

pytestmark = pytest.mark.gpu
H = 1326
# searches whose leaf values come from a network: how far product and oracle may sit apart on the
# entries the oracle determines, in tolerances (measured on the MI355X; see tests/parity.py)
NETWORK_FACTOR = 5.0      # largest seen: 2.4


@pytest.fixture(scope="module")
def K():
    from poker2_amd import chance_node_helper as M
    from poker2_amd import _lib
    assert _lib.hip_is_available(), "libp2hip.so / GPU missing"
    return M


def inputs(rng, b, ks):
    boards = np.full((b, 5), -1, dtype=np.int64)
    for i in range(b):
        k = ks[i % len(ks)]
        boards[i, :k] = random_boards(rng, 1, k)[0] if k else []
    pre = rng.gamma(0.5, size=(b, 2, H)).astype(np.float32)
    pre /= pre.sum(-1, keepdims=True)
    return boards, pre


def test_expand_matches_oracle_mixed_streets(K):
    rng = np.random.default_rng(5)
    boards, pre = inputs(rng, 9, [4, 3, 4, 0])
    pre[1, 0] = 0.0                      # dead range -> uniform fallback on every sample
    pre[2, 1] = 0.0
    pre[2, 1, 7] = 1.0                   # delta range -> dead on the samples that block it
    roots = np.array([8, 1, 2, 5, 0, 3])
    post, bs, lookup, offsets = K.chance_expand(torch.from_numpy(pre).cuda(), torch.from_numpy(roots).cuda(),
                                                torch.from_numpy(boards).cuda())
    e_post, e_bs, e_lookup = OCH.expand(pre[roots], boards[roots])
    assert torch.equal(bs.cpu(), torch.from_numpy(e_bs))                 # integer outputs: exact
    assert torch.equal(lookup.cpu(), torch.from_numpy(e_lookup))
    assert offsets.cpu().tolist() == np.concatenate([[0], np.cumsum(np.bincount(e_lookup))]).tolist()
    got = post.cpu().numpy()
    assert ((got == 0) == (e_post == 0)).all()                           # the mask is exact
    np.testing.assert_allclose(got, e_post, rtol=1e-5, atol=1e-9)        # float32 tolerance 1e-5 relative


def _expand_through_abi(pre, roots, boards, offset_floats, claimed_cards=None):
    """p2hip_chance_expand with the output `offset_floats` floats into a buffer: 0 keeps it 16-byte
    aligned (whole-line kernel), 2 leaves it 8-byte aligned (row-wise kernel).  `claimed_cards`: size
    the offsets and the buffers for that many cards on every board, whatever the boards hold."""
    from poker2_amd import _lib
    b = roots.numel()
    on_board = (boards[roots] >= 0).sum(1) if claimed_cards is None else torch.full((b,), claimed_cards, device=pre.device)
    offsets = torch.zeros(b + 1, dtype=torch.int64, device=pre.device)
    offsets[1:] = torch.cumsum(52 - on_board, 0)
    total = int(offsets[-1])
    buf = torch.full((total * 2 * H + 8,), float("nan"), device=pre.device)
    post = buf[offset_floats:offset_floats + total * 2 * H]
    bs = torch.full((total, 5), -7, dtype=torch.int64, device=pre.device)
    lookup = torch.full((total,), -7, dtype=torch.int64, device=pre.device)
    _lib.call("p2hip_chance_expand", _lib.ptr(pre), _lib.ptr(roots), _lib.ptr(boards), b, _lib.ptr(offsets),
              pre.shape[0], total, post.data_ptr(), _lib.ptr(bs), _lib.ptr(lookup), _lib.stream_ptr())
    torch.cuda.synchronize()
    assert torch.isnan(buf[:offset_floats]).all() and torch.isnan(buf[offset_floats + total * 2 * H:]).all()
    return post.view(total, 2, H), bs, lookup


@pytest.mark.parametrize("n", [5, 261, 1030])
def test_expand_whole_line_and_row_wise_kernels_agree_with_the_oracle(K, n):
    """Both forms of the expansion (16-byte aligned buffers -> whole 128-byte lines; 8-byte aligned ->
    rows as float2) on mixed boards: bit-identical to each other, and the oracle's samples to 1e-5.
    261 and 1030 states take runs of 13 cards per workgroup and end in a short group of states."""
    rng = np.random.default_rng(50 + n)
    boards, pre = inputs(rng, n, [4, 3, 4, 0, 4])
    pre[1, 0] = 0.0
    pre[2, 1] = 0.0
    pre[2, 1, 7] = 1.0
    roots = rng.permutation(n)[: max(n - 3, 1)]
    tp, tr, tb = torch.from_numpy(pre).cuda(), torch.from_numpy(roots).cuda(), torch.from_numpy(boards).cuda()
    wide = _expand_through_abi(tp, tr, tb, 0)
    narrow = _expand_through_abi(tp, tr, tb, 2)
    for x, y in zip(wide, narrow):
        assert torch.equal(x, y)
    e_post, e_bs, e_lookup = OCH.expand(pre[roots], boards[roots])
    assert torch.equal(wide[1].cpu(), torch.from_numpy(e_bs))
    assert torch.equal(wide[2].cpu(), torch.from_numpy(e_lookup))
    got = wide[0].cpu().numpy()
    assert ((got == 0) == (e_post == 0)).all()
    np.testing.assert_allclose(got, e_post, rtol=1e-5, atol=1e-9)


def test_mean_matches_oracle_and_ragged_counts(K):
    rng = np.random.default_rng(6)
    counts = np.array([48, 49, 0, 52, 1])
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    hv = rng.standard_normal((int(offsets[-1]), 2, H)).astype(np.float32)
    got = K.chance_mean(torch.from_numpy(hv).cuda(), torch.from_numpy(offsets).cuda()).cpu().numpy()
    lookup = np.repeat(np.arange(5), counts)
    exp = OCH.mean_by_root(hv, lookup, 5)
    np.testing.assert_allclose(got, exp, rtol=1e-5, atol=1e-6)
    assert not got[2].any()


class EchoModel:
    def eval(self):
        pass

    def __call__(self, f):
        return SimpleNamespace(hand_values=f.beliefs.view(-1, 2, H))


class BoardModel:
    """Values from the board's rank sum only (tests/test_chance_node_helper.py:78-117)."""

    def eval(self):
        pass

    def __call__(self, f):
        ranks = torch.where(f.board >= 0, (f.board % 13).float(), torch.zeros_like(f.board, dtype=torch.float32))
        v = ranks.sum(dim=1, keepdim=True) % H
        return SimpleNamespace(hand_values=v.unsqueeze(1).expand(-1, 2, H).contiguous())


@pytest.mark.parametrize("model_name", ["echo", "board"])
def test_helper_matches_oracle(K, model_name):
    rng = np.random.default_rng(8)
    b = 7
    boards, pre = inputs(rng, b, [4, 4, 3])
    roots = np.array([6, 0, 3, 4])
    dev = torch.device("cuda")
    model = EchoModel() if model_name == "echo" else BoardModel()
    helper = K.ChanceNodeHelper(dev, torch.float32, 2, model, autocast_dtype=None)
    feats = K.MLPFeatures(context=torch.zeros(b, 1, device=dev), street=torch.zeros(b, dtype=torch.long, device=dev),
                          to_act=torch.zeros(b, dtype=torch.long, device=dev),
                          board=torch.from_numpy(boards).to(dev), beliefs=torch.zeros(b, 2 * H, device=dev))
    got = helper.single_card_chance_values(torch.from_numpy(roots).to(dev), feats, torch.from_numpy(pre).to(dev),
                                           torch.from_numpy(boards).to(dev))

    def np_model(context, street, to_act, board, beliefs):
        if model_name == "echo":
            return beliefs.reshape(-1, 2, H)
        v = (np.where(board >= 0, board % 13, 0).sum(axis=1) % H).astype(np.float32)
        return np.broadcast_to(v[:, None, None], (board.shape[0], 2, H))
    exp = OCH.single_card_chance_values(roots, np.zeros((b, 1)), np.zeros(b), np.zeros(b), pre, boards, np_model)
    assert got.shape == (4, 2, H) and got.dtype == torch.float32
    np.testing.assert_allclose(got.cpu().numpy(), exp, rtol=1e-5, atol=1e-7)


def test_helper_edge_cases(K):
    dev = torch.device("cuda")
    helper = K.ChanceNodeHelper(dev, torch.float32, 2, EchoModel(), autocast_dtype=None)
    empty = K.MLPFeatures(context=torch.zeros(0, 1, device=dev), street=torch.zeros(0, dtype=torch.long, device=dev),
                          to_act=torch.zeros(0, dtype=torch.long, device=dev),
                          board=torch.zeros(0, 5, dtype=torch.long, device=dev), beliefs=torch.zeros(0, 2 * H, device=dev))
    out = helper.single_card_chance_values(torch.zeros(0, dtype=torch.long, device=dev), empty,
                                           torch.zeros(0, 2, H, device=dev), torch.zeros(0, 5, dtype=torch.long, device=dev))
    assert out.shape == (0, 2, H)
    full = torch.arange(5, device=dev)[None]                 # a river board has no chance card left
    with pytest.raises(ValueError):
        K.chance_expand(torch.rand(1, 2, H, device=dev), torch.zeros(1, dtype=torch.long, device=dev), full)
    out = helper.flop_chance_values(torch.zeros(0, dtype=torch.long, device=dev), empty, torch.zeros(0, 2, H, device=dev))
    assert out.shape == (0, 2, H)
    with pytest.raises(IndexError):                          # a state index beyond the ranges is refused on the host
        K.flop_expand(torch.rand(2, 2, H, device=dev), torch.tensor([2], device=dev), torch.tensor([[0, 1, 2]], device=dev))
    with pytest.raises(IndexError):                          # so is a permutation that points outside the hands
        K.perm_mean(torch.rand(1, 1, 2, H, device=dev), torch.full((1, H), H, device=dev), torch.ones(1, device=dev))
    # the fixed-count fast path gives the same samples
    rng = np.random.default_rng(9)
    boards, pre = inputs(rng, 3, [4])
    a = K.chance_expand(torch.from_numpy(pre).cuda(), torch.arange(3).cuda(), torch.from_numpy(boards).cuda())
    b = K.chance_expand(torch.from_numpy(pre).cuda(), torch.arange(3).cuda(), torch.from_numpy(boards).cuda(),
                        cards_on_board=4)
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    # a state index outside the ranges is refused on the host ...
    with pytest.raises(IndexError):
        K.chance_expand(torch.from_numpy(pre).cuda(), torch.tensor([3]).cuda(), torch.from_numpy(boards).cuda())
    # ... and a claimed card count above a board's real one (3 cards dealt, 4 claimed: 49 samples
    # where 48 were sized) cannot make the kernel write past the buffers: it stops at their end
    boards3 = boards.copy()
    boards3[1, 3] = -1
    boards3[2, 3] = -1                                       # the last state's 49th sample would lie past the end
    c = K.chance_expand(torch.from_numpy(pre).cuda(), torch.arange(3).cuda(), torch.from_numpy(boards3).cuda(),
                        cards_on_board=4)
    torch.cuda.synchronize()
    assert c[0].shape[0] == 3 * 48 and int(c[3][-1]) == 3 * 48          # offsets and buffers as claimed
    assert torch.equal(c[0][:48], a[0][:48]) and torch.equal(c[2][:48], a[2][:48])
    assert int(c[2].max()) <= 2 and int(c[2].min()) >= 0
    for offset in (0, 2):                                    # both kernels, with guard floats around the output
        g = _expand_through_abi(torch.from_numpy(pre).cuda(), torch.arange(3).cuda(), torch.from_numpy(boards3).cuda(),
                                offset, claimed_cards=4)
        assert torch.equal(g[0][:48], a[0][:48])


# ---- turn subgame: street-end leaves valued through the chance node + a small network --------
def numpy_mlp(net):
    ws = [(l.weight.detach().cpu().numpy().astype(np.float32), l.bias.detach().cpu().numpy().astype(np.float32))
          for l in net.linears]

    def fn(context, street, to_act, board, beliefs):
        onehot = np.zeros((board.shape[0], 52), np.float32)
        i, j = np.nonzero(board >= 0)
        onehot[i, board[i, j]] = 1.0
        x = np.concatenate([beliefs.astype(np.float32), onehot], axis=1)
        for k, (w, b) in enumerate(ws):
            x = x @ w.T + b
            if k < len(ws) - 1:
                x = np.maximum(x, 0.0)
        return x.reshape(-1, 2, H)
    return fn


@pytest.mark.parametrize("fused,streets", [(True, (2, 2)), (False, (2, 2)), (True, (3, 2, 2, 3))])
def test_turn_subgame_with_chance_leaves_matches_oracle(K, fused, streets):
    from oracle import cfr as OCFR
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.leaf_models import ChanceLeafModel, RangeBoardMLP
    from poker2_amd.tree import RootStates
    from tests.helpers import random_ranges
    from tests import parity as PAR
    from tests.helpers import tree_as_dict
    rng = np.random.default_rng(12)
    n, iters = len(streets), 5
    streets = np.array(streets)
    boards = random_boards(rng, n, 5)
    boards[streets == 2, 4] = -1                      # turn roots: the river card is still to come
    beliefs = random_ranges(rng, boards)
    roots = RootStates.at_round_start(streets, np.full(n, 200), np.tile([[800, 800]], (n, 1)), boards,
                                      button=np.arange(n) % 2)
    cfg = river_dcfr_config(n, iterations=iters, depth=16, dcfr_delay=0)
    dev = torch.device("cuda")
    net = RangeBoardMLP(hidden=64, layers=2, seed=3).to(dev)
    with torch.no_grad():
        for lin in net.linears:                       # orthogonal rows of a 2704-wide input give tiny outputs;
            lin.weight.mul_(4.0)                      # scale them up so leaf values matter to the strategy
    model = ChanceLeafModel(net, dev)
    ev = HipSparseCFREvaluator(model, dev, cfg, fused_iteration=fused, max_raises=1)
    ev.initialize_subgame(roots, np.arange(n), torch.from_numpy(beliefs))
    ev.prepare_search(t_sample=torch.full((ev.total_nodes,), -1, dtype=torch.long))
    tree = ev.tree
    n_turn, n_river = int((streets == 2).sum()), int((streets == 3).sum())
    assert ev.model_indices.numel() == 7 * n_turn and tree.showdown_mask.sum() == 7 * n_river
    mlp = numpy_mlp(net)
    node_board = tree.board[tree.root_index]
    street, to_act = tree.state["street"], tree.state["to_act"]

    def leaf_fn(bel, rows):
        k = len(rows)
        return OCH.single_card_chance_values(np.arange(k), np.zeros((k, 1), np.float32), street[rows], to_act[rows],
                                             bel[rows], node_board[rows], mlp)
    orc = OCFR.OracleCFR(tree_as_dict(tree), boards, beliefs, cfr_iterations=iters, leaf_value_fn=leaf_fn,
                         t_sample_roots=np.full(n, -1, dtype=np.int64), fused_variant=True)
    orc.prepare()
    # The network runs through hipBLASLt here and numpy there, so leaf values differ by GEMM summation
    # order, a few roundings of the network's output.  Which entries of the state that leaves open is
    # measured on the oracle (tests/parity.py: twins that start a few roundings away); every other
    # entry is held to NETWORK_FACTOR x (1e-5 relative + parity.ATOL).
    pack = PAR.OracleWithTwins(orc, seed=12, n_twins=2, amp=3e-7)
    PAR.compare_free(PAR.state_of(ev), pack, factor=NETWORK_FACTOR, kind="free running, network at the leaves", what="after the preparation step: ")
    assert np.abs(orc.latest_values[orc.model_indices]).max() > 1e-3     # the network's values are not trivial
    for t in range(iters):
        ev.cfr_iteration(t)
        pack.cfr_iteration(t)
        rep = PAR.compare_free(PAR.state_of(ev), pack, factor=NETWORK_FACTOR, kind="free running, network at the leaves", what=f"t={t}: ")
        print(f"t={t}: worst determined entry {PAR.worst_of(rep):.2f} tolerances, largest exempt share "
              f"{max(r['exempt'] for r in rep.values()):.1e}")


def test_helper_matches_vectors_from_the_reference_helper(K, golden_dir):
    """The HIP path against tests/golden/chance_golden.npz (written by running the reference's own
    ChanceNodeHelper.single_card_chance_values): bit-for-bit sample order is implied by the mean
    of a board-dependent network; values within float32 1e-5 relative."""
    g = np.load(str(golden_dir) + "/chance_golden.npz")
    board, pre, roots = g["board"], g["pre_beliefs"], g["root_indices"]
    n = board.shape[0]
    dev = torch.device("cuda")

    class BoardAndRange:
        def eval(self):
            pass

        def __call__(self, f):
            b = f.beliefs.view(-1, 2, H).float()
            ranks = torch.where(f.board >= 0, (f.board % 13).float(), torch.zeros_like(f.board, dtype=torch.float32))
            return SimpleNamespace(hand_values=b * (1.0 + ranks.sum(dim=1) / 100.0)[:, None, None])
    feats = K.MLPFeatures(context=torch.zeros(n, 1, device=dev), street=torch.full((n,), 3, dtype=torch.long, device=dev),
                          to_act=torch.zeros(n, dtype=torch.long, device=dev), board=torch.from_numpy(board).to(dev),
                          beliefs=torch.zeros(n, 2 * H, device=dev))
    for name, model in (("echo", EchoModel()), ("board_and_range", BoardAndRange())):
        helper = K.ChanceNodeHelper(dev, torch.float32, 2, model, autocast_dtype=None)
        got = helper.single_card_chance_values(torch.from_numpy(roots).to(dev), feats, torch.from_numpy(pre).to(dev),
                                               torch.from_numpy(board).to(dev))
        np.testing.assert_allclose(got.cpu().numpy(), g[name], rtol=1e-5, atol=1e-8)


# ---- three-card (flop) chance node -------------------------------------------------------------
def test_flop_expand_matches_oracle(K):
    rng = np.random.default_rng(21)
    pre = rng.gamma(0.5, size=(5, 2, H)).astype(np.float32)
    pre /= pre.sum(-1, keepdims=True)
    pre[1, 0] = 0.0                      # dead range -> uniform over the 1176 hands left
    pre[3, 1] = 0.0
    pre[3, 1, 0] = 1.0                   # delta on hand (0,1): dead on flops holding card 0 or 1
    flops = np.stack([rng.permutation(52)[:3] for _ in range(37)]).astype(np.int64)   # any card order, > 16 flops
    flops[0] = [0, 13, 26]
    flops[1] = [5, 1, 40]
    roots = np.array([4, 1, 3, 3, 0])
    got = K.flop_expand(torch.from_numpy(pre).cuda(), torch.from_numpy(roots).cuda(),
                        torch.from_numpy(flops).cuda()).cpu().numpy()
    exp = OCH.flop_expand(pre[roots], flops)
    assert got.shape == (5, 37, 2, H)
    assert ((got == 0) == (exp == 0)).all()                              # the mask is exact
    np.testing.assert_allclose(got, exp, rtol=1e-5, atol=1e-9)           # float32 tolerance 1e-5 relative
    np.testing.assert_allclose(got.sum(-1), 1.0, rtol=1e-5)
    # no flops: an empty result, no launch
    assert K.flop_expand(torch.from_numpy(pre).cuda(), torch.from_numpy(roots).cuda(),
                         torch.zeros(0, 3, dtype=torch.long).cuda()).shape == (5, 0, 2, H)


@pytest.mark.parametrize("n,k", [(3, 5), (13, 37), (70, 129)])
def test_flop_expand_whole_line_and_row_wise_kernels_agree(K, n, k):
    """p2hip_flop_expand into a 16-byte aligned and into an 8-byte aligned buffer: bit-identical, and equal
    to the oracle to 1e-5 (70 x 129 takes eight flops per workgroup, the others four)."""
    from poker2_amd import _lib
    rng = np.random.default_rng(n * 100 + k)
    pre = rng.gamma(0.5, size=(n, 2, H)).astype(np.float32)
    pre /= pre.sum(-1, keepdims=True)
    pre[1, 0] = 0.0
    flops = np.stack([rng.permutation(52)[:3] for _ in range(k)]).astype(np.int64)
    flops[2] = [9, 9, 30]                # not three distinct cards: an all-zero sample
    tp, tf = torch.from_numpy(pre).cuda(), torch.from_numpy(flops).cuda()
    roots = torch.arange(n).cuda()
    outs = []
    for offset in (0, 2):
        buf = torch.full((n * k * 2 * H + 8,), float("nan"), device="cuda")
        out = buf[offset:offset + n * k * 2 * H]
        _lib.call("p2hip_flop_expand", _lib.ptr(tp), _lib.ptr(roots), n, _lib.ptr(tf), k, out.data_ptr(),
                  _lib.stream_ptr())
        torch.cuda.synchronize()
        assert torch.isnan(buf[:offset]).all() and torch.isnan(buf[offset + n * k * 2 * H:]).all()
        outs.append(out.view(n, k, 2, H))
    assert torch.equal(outs[0], outs[1])
    ok = np.ones(k, dtype=bool)
    ok[2] = False
    exp = OCH.flop_expand(pre, flops[ok])
    got = outs[0].cpu().numpy()
    assert (got[:, 2] == 0).all()
    assert ((got[:, ok] == 0) == (exp == 0)).all()
    np.testing.assert_allclose(got[:, ok], exp, rtol=1e-5, atol=1e-9)


@pytest.mark.parametrize("lead", [(5,), (3, 2), (2, 3, 2), (0, 2)])
def test_avg_over_perms_any_leading_shape(K, lead):
    """The reference's ``_avg_over_perms`` (chance_node_helper.py:17-27) on values of any leading
    shape, an odd number of rows included."""
    rng = np.random.default_rng(31)
    perms = OCH.combo_suit_perms()[rng.permutation(24)[:6]]
    hv = rng.standard_normal(lead + (H,)).astype(np.float32)
    exp = np.mean([hv[..., q] for q in perms], axis=0, dtype=np.float64) if hv.size else hv
    got = K._avg_over_perms(torch.from_numpy(hv).cuda(), torch.from_numpy(perms).cuda())
    assert got.shape == hv.shape
    np.testing.assert_allclose(got.cpu().numpy(), exp, rtol=1e-5, atol=2e-6)


@pytest.mark.parametrize("n_perms,kind", [(1, "suits"), (6, "suits"), (8, "suits"), (24, "suits"),
                                          (6, "any"), (6, "one_off"), (3, "not_bijective")])
def test_perm_mean_matches_numpy(K, n_perms, kind):
    """Suit permutations (up to 8 of them sit in registers, more in LDS), arbitrary permutations of
    the hands, a suit permutation with two hands swapped, and a table that is no permutation at all
    (every hand reads the same source): all are plain gathers."""
    rng = np.random.default_rng(22 + n_perms + len(kind))
    perms = OCH.combo_suit_perms()[rng.permutation(24)[:n_perms]].copy()
    if kind == "any":
        perms[2] = rng.permutation(H)
    elif kind == "one_off":
        perms[4, [700, 701]] = perms[4, [701, 700]]
    elif kind == "not_bijective":
        perms[1] = perms[1][0]
    hv = rng.standard_normal((3, 11, 2, H)).astype(np.float32)
    w = rng.random(11).astype(np.float32)
    exp = np.zeros((3, 2, H))
    for k in range(11):
        exp += w[k] * np.mean([hv[:, k][..., q] for q in perms], axis=0, dtype=np.float64)
    got = K.perm_mean(torch.from_numpy(hv).cuda(), torch.from_numpy(perms).cuda(), torch.from_numpy(w).cuda())
    np.testing.assert_allclose(got.cpu().numpy(), exp, rtol=1e-5, atol=2e-6)
    # accumulation onto an earlier result
    again = K.perm_mean(torch.from_numpy(hv).cuda(), torch.from_numpy(perms).cuda(), torch.from_numpy(w).cuda(),
                        out=got.clone())
    np.testing.assert_allclose(again.cpu().numpy(), 2 * exp, rtol=1e-5, atol=4e-6)
    # many states: one workgroup per (state, player) walks all flops and writes the result itself
    hv = rng.standard_normal((1100, 3, 2, H)).astype(np.float32)
    w = rng.random(3).astype(np.float32)
    exp = np.zeros((1100, 2, H))
    for k in range(3):
        exp += w[k] * np.mean([hv[:, k][..., q] for q in perms], axis=0, dtype=np.float64)
    base = rng.standard_normal((1100, 2, H)).astype(np.float32)
    got = K.perm_mean(torch.from_numpy(hv).cuda(), torch.from_numpy(perms).cuda(), torch.from_numpy(w).cuda(),
                      out=torch.from_numpy(base).cuda())
    np.testing.assert_allclose(got.cpu().numpy(), base + exp, rtol=1e-5, atol=4e-6)


def test_helper_flop_cache_matches_the_reference_cache(K, golden_dir):
    g = np.load(str(golden_dir) + "/flop_chance_golden.npz")
    helper = K.ChanceNodeHelper(torch.device("cuda"), torch.float32, 2, EchoModel(), autocast_dtype=None)
    assert np.array_equal(helper.flop_id_to_canonical.cpu().numpy(), g["flop_id_to_canonical"].astype(np.int64))
    assert np.array_equal(helper.flop_id_to_count.cpu().numpy(), g["flop_id_to_count"].astype(np.int64))
    assert np.array_equal(helper.flop_to_canon.cpu().numpy(), g["flop_to_canon"].astype(np.int64))
    assert np.array_equal(helper.combo_perm.cpu().numpy(), g["combo_perm"].astype(np.int64))
    assert np.array_equal(helper.board_to_flop_id[3, 17, 40:52].cpu().numpy(), g["board_to_flop_id_sample"].astype(np.int64))
    assert helper.total_flop_count == 22100


class SuitAwareModel:
    """torch twin of the network in tests/golden/gen_flop_chance_golden.py."""

    def eval(self):
        pass

    def __call__(self, f):
        b = f.beliefs.view(-1, 2, H).float()
        w = 1.0 + (f.board[:, 0] // 13).float() / 10.0 + (f.board[:, 2] % 13).float() / 100.0
        h = (torch.arange(H, device=b.device) % 7).float() * 0.001
        return SimpleNamespace(hand_values=b * w[:, None, None]
                               + h[None, None, :] * torch.tensor([1.0, 2.0], device=b.device)[None, :, None])


@pytest.mark.parametrize("mode,sample,nperm", [("all", 0, 0), ("all_perm6", 0, 6), ("sample256_perm6", 256, 6)])
def test_helper_flop_values_match_vectors_from_the_reference_helper(K, golden_dir, mode, sample, nperm):
    """flop_chance_values against tests/golden/flop_chance_golden.npz (written by running the
    reference's helper).  The draws come from a CPU generator with the fixture's seed, as in the
    run that wrote it, so the sampled modes see the same flops and permutations."""
    g = np.load(str(golden_dir) + "/flop_chance_golden.npz")
    pre, roots = g["pre_beliefs"], g["root_indices"]
    n = pre.shape[0]
    dev = torch.device("cuda")
    feats = K.MLPFeatures(context=torch.zeros(n, 1, device=dev), street=torch.zeros(n, dtype=torch.long, device=dev),
                          to_act=torch.zeros(n, dtype=torch.long, device=dev),
                          board=torch.full((n, 5), -1, dtype=torch.long, device=dev), beliefs=torch.zeros(n, 2 * H, device=dev))
    for name, model in (("echo", EchoModel()), ("suit_aware", SuitAwareModel())):
        gen = torch.Generator(device="cpu")
        gen.manual_seed(int(g["seed"]))
        helper = K.ChanceNodeHelper(dev, torch.float32, 2, model, generator=gen, autocast_dtype=None)
        helper.FLOP_SAMPLE_SIZE, helper.NUM_PERM_SAMPLES = sample, nperm
        got = helper.flop_chance_values(torch.from_numpy(roots).to(dev), feats, torch.from_numpy(pre).to(dev))
        assert got.shape == (2, 2, H) and got.dtype == torch.float32
        np.testing.assert_allclose(got.cpu().numpy(), g[f"{name}_{mode}"], rtol=1e-5, atol=1e-7, err_msg=f"{name} {mode}")


def test_helper_flop_values_device_generator_is_unbiased_sample(K):
    """Default settings (256 drawn classes, 6 drawn permutations, device generator): the estimate
    stays close to the full enumeration for a smooth network and repeats under the same seed."""
    rng = np.random.default_rng(31)
    pre = rng.gamma(0.5, size=(2, 2, H)).astype(np.float32)
    pre /= pre.sum(-1, keepdims=True)
    dev = torch.device("cuda")
    feats = K.MLPFeatures(context=torch.zeros(2, 1, device=dev), street=torch.zeros(2, dtype=torch.long, device=dev),
                          to_act=torch.zeros(2, dtype=torch.long, device=dev),
                          board=torch.full((2, 5), -1, dtype=torch.long, device=dev), beliefs=torch.zeros(2, 2 * H, device=dev))
    outs = []
    for _ in range(2):
        gen = torch.Generator(device=dev)
        gen.manual_seed(7)
        helper = K.ChanceNodeHelper(dev, torch.float32, 2, SuitAwareModel(), generator=gen, autocast_dtype=None)
        outs.append(helper.flop_chance_values(torch.arange(2, device=dev), feats, torch.from_numpy(pre).to(dev)))
    assert torch.equal(outs[0], outs[1])
    helper.FLOP_SAMPLE_SIZE, helper.NUM_PERM_SAMPLES = 0, 0
    full = helper.flop_chance_values(torch.arange(2, device=dev), feats, torch.from_numpy(pre).to(dev))
    # total mass per player is preserved by both; the sampled estimate of it is within a few percent
    np.testing.assert_allclose(outs[0].sum(-1).cpu().numpy(), full.sum(-1).cpu().numpy(), rtol=0.05)


def test_preflop_subgame_with_flop_leaves_matches_oracle(K):
    """Preflop roots: the leaves that close the betting round are valued by the flop chance node
    (all 1755 classes, all 24 permutations, so nothing is drawn) in front of a small network."""
    from oracle import cfr as OCFR
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.leaf_models import ChanceLeafModel, RangeBoardMLP
    from poker2_amd.tree import RootStates
    from tests import parity as PAR
    from tests.helpers import tree_as_dict
    rng = np.random.default_rng(14)
    n, iters = 2, 3
    boards = np.full((n, 5), -1, dtype=np.int64)
    beliefs = rng.gamma(0.5, size=(n, 2, H)).astype(np.float32)
    beliefs /= beliefs.sum(-1, keepdims=True)
    roots = RootStates.preflop(n, starting_stacks=1000, button=np.arange(n) % 2)
    cfg = river_dcfr_config(n, iterations=iters, depth=2, dcfr_delay=0)
    dev = torch.device("cuda")
    net = RangeBoardMLP(hidden=64, layers=2, seed=5).to(dev)
    with torch.no_grad():
        for lin in net.linears:
            lin.weight.mul_(4.0)
    model = ChanceLeafModel(net, dev)
    model.helper.FLOP_SAMPLE_SIZE, model.helper.NUM_PERM_SAMPLES = 0, 0
    ev = HipSparseCFREvaluator(model, dev, cfg, fused_iteration=True, max_raises=1)
    ev.initialize_subgame(roots, np.arange(n), torch.from_numpy(beliefs))
    ev.prepare_search(t_sample=torch.full((ev.total_nodes,), -1, dtype=torch.long))
    tree = ev.tree
    rows_model = ev.model_indices.cpu().numpy()
    closes = tree.new_street_mask[rows_model]
    assert closes.any() and (~closes).any()           # both kinds of leaf: round closed (flop to come) and mid-round
    mlp = numpy_mlp(net)
    street, to_act = tree.state["street"], tree.state["to_act"]
    canonical, count, _ = OCH.canonical_flops()
    perms = OCH.combo_suit_perms()

    def leaf_fn(bel, rows):
        rows = np.asarray(rows)
        out = np.zeros((len(rows), 2, H), np.float32)
        flop = tree.new_street_mask[rows]
        if flop.any():
            r = rows[flop]
            out[flop] = OCH.flop_chance_values(np.arange(len(r)), np.zeros((len(r), 1), np.float32), street[r],
                                               to_act[r], bel[r], mlp, canonical, count, perms)
        if (~flop).any():
            r = rows[~flop]
            out[~flop] = mlp(None, street[r], to_act[r], np.full((len(r), 5), -1), bel[r].reshape(len(r), -1))
        return out
    orc = OCFR.OracleCFR(tree_as_dict(tree), boards, beliefs, cfr_iterations=iters, leaf_value_fn=leaf_fn,
                         t_sample_roots=np.full(n, -1, dtype=np.int64), fused_variant=True)
    orc.prepare()
    pack = PAR.OracleWithTwins(orc, seed=14, n_twins=2, amp=3e-7)      # as in the turn test above
    PAR.compare_free(PAR.state_of(ev), pack, factor=NETWORK_FACTOR, kind="free running, network at the leaves", what="after the preparation step: ")
    assert np.abs(orc.latest_values[orc.model_indices]).max() > 1e-3
    for t in range(iters):
        ev.cfr_iteration(t)
        pack.cfr_iteration(t)
        rep = PAR.compare_free(PAR.state_of(ev), pack, factor=NETWORK_FACTOR, kind="free running, network at the leaves", what=f"t={t}: ")
        print(f"t={t}: worst determined entry {PAR.worst_of(rep):.2f} tolerances, largest exempt share "
              f"{max(r['exempt'] for r in rep.values()):.1e}")


def test_orbit_mean_equals_the_mean_over_all_24_permutations(K):
    """The class-mean shortcut against the literal mean over the 24 permuted copies (numpy, fp64)
    and against the generic kernel fed with the full permutation table."""
    rng = np.random.default_rng(71)
    perms = OCH.combo_suit_perms()
    classes = {tuple(sorted(set(perms[:, h].tolist()))) for h in range(H)}
    assert len(classes) == 169 and sorted({len(c) for c in classes}) == [4, 6, 12]   # suited, pairs, offsuit
    for b, k in ((3, 11), (1100, 2)):            # flops shared out over workgroups / one workgroup per (state, player)
        hv = rng.standard_normal((b, k, 2, H)).astype(np.float32)
        w = rng.random(k).astype(np.float32)
        exp = np.zeros((b, 2, H))
        for f in range(k):
            exp += w[f] * np.mean([hv[:, f][..., q] for q in perms], axis=0, dtype=np.float64)
        t_hv, t_w = torch.from_numpy(hv).cuda(), torch.from_numpy(w).cuda()
        got = K.orbit_mean(t_hv, t_w)
        np.testing.assert_allclose(got.cpu().numpy(), exp, rtol=1e-5, atol=2e-6)
        generic = K.perm_mean(t_hv, torch.from_numpy(perms).cuda(), t_w)
        np.testing.assert_allclose(got.cpu().numpy(), generic.cpu().numpy(), rtol=1e-5, atol=2e-6)
        base = torch.from_numpy(rng.standard_normal((b, 2, H)).astype(np.float32)).cuda()
        again = K.orbit_mean(t_hv, t_w, out=base.clone())
        np.testing.assert_allclose(again.cpu().numpy(), base.cpu().numpy() + exp, rtol=1e-5, atol=4e-6)


# ---- the expansion written straight into the network's input matrix ---------------------------
@pytest.mark.parametrize("n", [6, 300])
def test_expansion_as_input_rows_equals_concatenation_and_cast(K, n):
    """``chance_expand(..., input_dtype=...)``: rows [ranges | one-hot of the sample's board] in float32 /
    bfloat16 / float16 against what the network's own ``forward`` builds from the plain expansion
    (scatter one-hot, concatenate, cast): bit for bit — the values are those of the plain expansion,
    which the oracle pins, and the casts round like torch's."""
    rng = np.random.default_rng(70 + n)
    boards, pre = inputs(rng, n, [4, 3, 4, 0, 4])
    pre[1, 0] = 0.0
    roots = torch.from_numpy(rng.permutation(n)[: max(n - 2, 1)]).cuda()
    tp, tb = torch.from_numpy(pre).cuda(), torch.from_numpy(boards).cuda()
    post, bs, lookup, offsets = K.chance_expand(tp, roots, tb)
    onehot = torch.zeros(bs.shape[0], 53, device="cuda")
    onehot.scatter_(1, torch.where(bs >= 0, bs, torch.full_like(bs, 52)), 1.0)
    want = torch.cat([post.reshape(post.shape[0], -1), onehot[:, :52]], dim=1)
    for dt in (torch.float32, torch.bfloat16, torch.float16):
        rows, bs2, lookup2, offsets2 = K.chance_expand(tp, roots, tb, input_dtype=dt)
        assert rows.dtype == dt and rows.shape == (post.shape[0], K.INPUT_ROW_WIDTH)
        assert torch.equal(rows, want.to(dt)), dt
        assert torch.equal(bs2, bs) and torch.equal(lookup2, lookup) and torch.equal(offsets2, offsets)


@pytest.mark.parametrize("autocast", [None, torch.bfloat16])
def test_helper_feeds_a_ranges_and_board_network_without_concatenation(K, autocast):
    """``single_card_chance_values`` with a network that declares its input as [ranges | board one-hot]
    (RangeBoardMLP): the expansion writes the input matrix, ``forward_input`` runs on it; same answer as the
    feature-bundle path (``forward``: scatter, concatenate, cast under autocast) — the same numbers reach the
    same GEMMs."""
    from poker2_amd.leaf_models import RangeBoardMLP
    rng = np.random.default_rng(77)
    n = 40
    boards, pre = inputs(rng, n, [4])
    dev = torch.device("cuda")
    net = RangeBoardMLP(hidden=64, layers=2, seed=5).to(dev)

    class Plain(torch.nn.Module):                      # the same network without the declaration
        def __init__(self, inner):
            super().__init__()
            self.inner = inner

        def forward(self, f):
            return self.inner(f)
    roots = torch.arange(n, device=dev)
    feats = K.MLPFeatures(context=torch.zeros(n, 4, device=dev), street=torch.full((n,), 2, device=dev),
                          to_act=torch.zeros(n, dtype=torch.long, device=dev), board=torch.from_numpy(boards).to(dev),
                          beliefs=torch.from_numpy(pre).to(dev).reshape(n, -1))
    tp, tb = torch.from_numpy(pre).to(dev), torch.from_numpy(boards).to(dev)
    direct = K.ChanceNodeHelper(dev, torch.float32, 2, net, autocast_dtype=autocast)
    bundle = K.ChanceNodeHelper(dev, torch.float32, 2, Plain(net), autocast_dtype=autocast)
    a = direct.single_card_chance_values(roots, feats, tp, tb)
    b = bundle.single_card_chance_values(roots, feats, tp, tb)
    c = direct.single_card_chance_values(roots, feats, tp, tb, cards_on_board=4, check_rows=False)
    assert torch.equal(a, b) and torch.equal(a, c)
    assert float(a.abs().max()) > 0


def test_a_wrong_card_count_claim_leaves_defined_rows(K):
    """With ``cards_on_board`` claimed and ``check_rows=False`` the outputs are sized on trust.  A board that
    holds more cards than claimed, a board without an empty slot and a row outside the table yield fewer
    samples than their share of the buffers: the rest of the share is zeros with ``root_lookup`` = the state,
    in every form of the expansion, so nothing uninitialised reaches the network."""
    rng = np.random.default_rng(78)
    boards, pre = inputs(rng, 5, [3])
    boards[1, 3] = 40 if 40 not in boards[1] else 41            # four cards where three are claimed
    boards[2] = np.array([0, 1, 2, 3, 4])                       # no empty slot
    roots = torch.tensor([0, 1, 2, 7, 4]).cuda()                # 7: outside the table
    tp, tb = torch.from_numpy(pre).cuda(), torch.from_numpy(boards).cuda()
    for kw in ({}, {"input_dtype": torch.float32}, {"input_dtype": torch.bfloat16}):
        for poison in (float("nan"), 3.0):
            # the caching allocator hands the poisoned block back to the call below
            width = 2 * H if not kw else K.INPUT_ROW_WIDTH
            junk = torch.full((5 * 49, width), poison, dtype=kw.get("input_dtype", torch.float32), device="cuda")
            del junk
            out, bs, lookup, offsets = K.chance_expand(tp, roots, tb, cards_on_board=3, check_rows=False, **kw)
            torch.cuda.synchronize()
            rows = out.reshape(5, 49, -1).float()
            assert bool(torch.isfinite(rows).all())
            assert float(rows[1, 48].abs().max()) == 0 and float(rows[1, :48, :2 * H].sum()) > 0     # 48 samples + one zero row
            assert float(rows[2].abs().max()) == 0 and float(rows[3].abs().max()) == 0                # nothing to expand
            assert lookup.view(5, 49).eq(torch.arange(5, device="cuda")[:, None]).all()
            assert float(rows[0, :, :2 * H].sum()) > 0 and float(rows[4, :, :2 * H].sum()) > 0
    # the row-wise kernel (8-byte aligned output) through the C ABI: the same
    g = _expand_through_abi(tp, roots, tb, 2, claimed_cards=3)
    assert bool(torch.isfinite(g[0]).all()) and float(g[0].view(5, 49, -1)[2].abs().max()) == 0
    assert g[2].view(5, 49).eq(torch.arange(5, device="cuda")[:, None]).all()
