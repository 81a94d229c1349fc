"""GPU parity of the single-card chance node (expansion + mean kernels and the
ChanceNodeHelper mirror) against the oracle, on the cases of the reference's
tests/test_chance_node_helper.py:426-590 and on seeded mixed-street inputs."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import chance as OCH
from tests.helpers import random_boards

pytestmark = pytest.mark.gpu
H = 1326


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
    with pytest.raises(NotImplementedError):
        helper.flop_chance_values()
    # the fixed-count fast path gives the same samples
    rng = np.random.default_rng(9)
    boards, pre = inputs(rng, 3, [4])
    a = K.chance_expand(torch.from_numpy(pre).cuda(), torch.arange(3).cuda(), torch.from_numpy(boards).cuda())
    b = K.chance_expand(torch.from_numpy(pre).cuda(), torch.arange(3).cuda(), torch.from_numpy(boards).cuda(),
                        cards_on_board=4)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


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
    from tests.test_gpu_evaluator import compare, tree_as_dict
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
    compare(ev, orc, rtol=2e-4, atol=2e-5)
    assert np.abs(orc.latest_values[orc.model_indices]).max() > 1e-3     # the network's values are not trivial
    # the network runs through hipBLASLt here and numpy there: leaf values differ by GEMM summation
    # order (~1e-6 relative) and regret matching divides by small regret sums, hence the wider bar
    for t in range(iters):
        ev.cfr_iteration(t)
        orc.cfr_iteration(t)
        compare(ev, orc, rtol=1e-3, atol=3e-4)


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
