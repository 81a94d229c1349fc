"""GPU parity of the steps either side of the search in data generation: feature encoding, bet
amounts, policy targets (kernels against the oracle on seeded inputs) and ``training_data`` of
the evaluator against vectors written by running the reference's evaluator
(tests/golden/training_data_golden.npz) and against the oracle on the same search."""
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import cards as OC
from oracle import cfr as OCFR
from oracle import chance as OCH
from oracle import datagen as ODG
from tests.test_oracle_datagen import BINS, case_settings, load_case, oracle_search_arguments, value_net_numpy

pytestmark = pytest.mark.gpu
H = 1326
DEV = "cuda"


class ValueNet:
    """torch twin of ``ValueNet`` in tests/golden/gen_training_data_golden.py."""
    enforce_zero_sum = False

    def eval(self):
        pass

    def __call__(self, f):
        b = f.beliefs.view(-1, 2, H).float()
        ranks = torch.where(f.board >= 0, (f.board % 13 + 1).float(), torch.zeros_like(f.board, dtype=torch.float32))
        w = (0.2 + 0.1 * f.context[:, 2] + 0.05 * f.context[:, 1] - 0.03 * f.context[:, 3]
             + 0.01 / 13.0 * ranks.sum(dim=1))
        opp = torch.flip(b, dims=[1])
        sign = torch.tensor([1.0, -1.0], device=b.device)[None, :, None]
        h = ((torch.arange(H, device=b.device) % 7).float() - 3.0) * 0.002
        return SimpleNamespace(hand_values=sign * 0.05 * w[:, None, None] * (H * opp - 1.0) + h[None, None, :])


def random_env(rng, m):
    street = rng.integers(0, 4, m)
    board = np.full((m, 5), -1, dtype=np.int64)
    for i in range(m):
        k = [0, 3, 4, 5][street[i]]
        board[i, :k] = rng.permutation(52)[:k]
    actions = rng.integers(0, 4, m)
    env = {"to_act": rng.integers(0, 2, m), "button": rng.integers(0, 2, m),
           "starting_stacks": rng.integers(0, 3, (m, 2)) * rng.integers(1, 30000, (m, 2)),
           "pot": rng.integers(0, 50000, m), "committed": rng.integers(0, 3, (m, 2)) * rng.integers(0, 500, (m, 2)),
           "stacks": rng.integers(0, 20000, (m, 2)), "actions_this_round": actions, "street": street,
           "board_indices": board, "last_board_indices": ODG.previous_board(street, actions, board)}
    return {k: v.astype(np.int64) for k, v in env.items()}


def as_namespace(env):
    return SimpleNamespace(**{k: torch.from_numpy(v).to(DEV) for k, v in env.items()})


def test_encode_matches_oracle_all_argument_forms():
    from poker2_amd.rebel_feature_encoder import RebelFeatureEncoder
    rng = np.random.default_rng(40)
    m = 777
    env = random_env(rng, m)
    bel = rng.random((m, 2, H)).astype(np.float32)
    enc = RebelFeatureEncoder(as_namespace(env))
    tb = torch.from_numpy(bel).to(DEV)
    pre = rng.random(m) < 0.5
    idx = rng.permutation(m)[:100]
    for kw_o, kw_p in (({}, {}), ({"pre_chance_node": True}, {"pre_chance_node": True}),
                       ({"pre_chance_node": pre}, {"pre_chance_node": torch.from_numpy(pre).to(DEV)}),
                       ({"pre_chance_node": pre, "indices": idx},
                        {"pre_chance_node": torch.from_numpy(pre).to(DEV), "indices": torch.from_numpy(idx).to(DEV)}),
                       ({"pre_chance_node": False, "indices": idx}, {"pre_chance_node": False, "indices": torch.from_numpy(idx)})):
        exp = ODG.encode(env, bel, **kw_o)
        got = enc.encode(tb, **kw_p)
        assert np.array_equal(got.context.cpu().numpy(), exp["context"])          # same float32 operations: exact
        assert np.array_equal(got.board.cpu().numpy(), exp["board"])
        assert np.array_equal(got.to_act.cpu().numpy(), exp["to_act"])
        assert np.array_equal(got.street.cpu().numpy(), exp["street"])
        assert np.array_equal(got.beliefs.cpu().numpy(), exp["beliefs"])
    empty = enc.encode(tb, indices=torch.zeros(0, dtype=torch.long, device=DEV))
    assert len(empty) == 0 and empty.context.shape == (0, 4)


def test_bet_amounts_match_oracle():
    from poker2_amd.evaluator import _TreeEnv
    rng = np.random.default_rng(41)
    m = 1000
    env = random_env(rng, m)
    for bins in ([0.5, 1.0], [0.33, 0.75, 1.5], [], [0.25, 0.5, 1.0, 2.0, 4.0]):
        ns = as_namespace(env)
        te = _TreeEnv(N=m, default_bet_bins=bins, legal_mask=None, **vars(ns))
        got, _ = te.legal_bins_amounts_and_mask()
        assert np.array_equal(got.cpu().numpy(), ODG.bet_amounts(env, bins)), bins    # int64: exact


def search_config(n, depth, iters, algo):
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.fused_cfr_hip import CFRType
    cfg = river_dcfr_config(n, iterations=iters, depth=depth, dcfr_delay=algo["delay"])
    z = cfg.search
    z.cfr_type = CFRType[algo["cfr_type"]]
    z.cfr_plus, z.cfr_avg = algo["cfr_plus"], algo["cfr_avg"]
    z.warm_start_iterations, z.warm_start_type, z.warm_start_multiplier = algo["warm"], algo["warm_type"], algo["warm_mult"]
    z.dcfr_alpha, z.dcfr_beta, z.dcfr_gamma = algo["alpha"], algo["beta"], algo["gamma"]
    z.dcfr_alpha_final, z.dcfr_beta_final, z.dcfr_gamma_final = algo["alpha_final"], algo["beta_final"], algo["gamma_final"]
    z.value_targets_from_final_policy = algo["final_policy_values"]
    return cfg


def linear_plus(case):
    """Linear CFR with CFR+: the base class clamps the accumulated regrets, the fused class (which
    the product follows) does not (fused_sparse_cfr_evaluator.py:503-507), so the two play
    different strategies and only a fused-class fixture applies."""
    algo = case_settings(case)[2]
    return algo["cfr_type"] == "linear" and algo["cfr_plus"]


def golden_evaluator(case, fused):
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.leaf_models import NetworkLeafModel
    from poker2_amd.tree import RootStates
    r = {k[5:]: v for k, v in case.items() if k.startswith("root/")}
    n = len(r["street"])
    roots = RootStates.from_env(SimpleNamespace(bb=100, **r), np.arange(n))
    depth, iters, algo = case_settings(case)
    cfg = search_config(n, depth, iters, algo)
    model = NetworkLeafModel(ValueNet(), DEV, enforce_zero_sum=algo["enforce_zero_sum"])
    ev = HipSparseCFREvaluator(model, torch.device(DEV), cfg, fused_iteration=fused)
    ev.initialize_subgame(roots, np.arange(n), torch.from_numpy(case["beliefs"]))
    ev.prepare_search(t_sample=torch.full((ev.total_nodes,), -1, dtype=torch.long))     # includes the warm start
    for t in range(algo["warm"], iters):
        ev.cfr_iteration(t)
    if ev.use_final_policy_values:
        ev.update_average_values_final()
    ev.chance_helper.FLOP_SAMPLE_SIZE, ev.chance_helper.NUM_PERM_SAMPLES = 0, 0
    WORST.clear()
    return ev, r


def batch_as_dict(b):
    out = {"features": {"context": b.features.context, "board": b.features.board, "to_act": b.features.to_act,
                        "street": b.features.street, "beliefs": b.features.beliefs},
           "legal_masks": b.legal_masks, "statistics": dict(b.statistics)}
    if b.value_targets is not None:
        out["value_targets"] = b.value_targets
    if b.policy_targets is not None:
        out["policy_targets"] = b.policy_targets

    def host(x):
        return {k: host(v) for k, v in x.items()} if isinstance(x, dict) else x.cpu().numpy()
    return host(out)


# Training targets sit behind a whole search (4-12 iterations of regret matching), so product and
# reference differ by accumulated roundings.  Exemptions are by cause, as in tests/parity.py: the
# oracle runs the same search, twice more from a state a few roundings away, and an entry of a target
# is exempt if either twin moves it by more than a third of the tolerance; every other entry is held
# to TARGET_FACTOR x (1e-5 relative + the absolute part below).  Largest seen on the MI355X: see the
# printed reports; the exempt share of a tensor is capped.
TARGET_ATOL = {"beliefs": 1e-7, "value_targets": 2e-6, "policy_targets": 1e-6}
TARGET_FACTOR = 5.0
TARGET_MAX_EXEMPT = 0.35
LOOP_FACTOR = 30.0     # largest seen: 13.3


def oracle_with_twins(case, ev, r, fused_variant=True, n_twins=2):
    """The oracle's training data of the case's search and that of `n_twins` perturbed twins."""
    from tests import parity as PAR
    from tests.helpers import tree_as_dict
    tree = tree_as_dict(ev.tree)
    tree.update({k: v for k, v in ev.tree.state.items() if k not in tree})
    env = ODG.tree_env(tree, r["board_indices"])

    def leaf_fn(beliefs, rows):
        f = ODG.encode(env, beliefs, pre_chance_node=tree["new_street_mask"], indices=rows)
        return value_net_numpy(f["context"], f["street"], f["to_act"], f["board"], f["beliefs"])
    _, iters, algo = case_settings(case)
    o = OCFR.OracleCFR(tree, r["board_indices"], case["beliefs"], cfr_iterations=iters, leaf_value_fn=leaf_fn,
                       t_sample_roots=np.full(ev.root_nodes, -1, dtype=np.int64), fused_variant=fused_variant,
                       **oracle_search_arguments(algo))
    o.prepare()
    pack = PAR.OracleWithTwins(o, n_twins=n_twins, amp=3e-7, seed=21)
    for t in range(algo["warm"], iters):
        pack.cfr_iteration(t)
    canonical, count, _ = OCH.canonical_flops()
    out = []
    for x in [pack.base] + pack.twins:
        if x.use_final_policy_values:
            x.update_average_values_final()
        out.append(ODG.training_data(x, env, BINS, value_net_numpy, flop_tables=(canonical, count, OCH.combo_suit_perms())))
    return out[0], out[1:]


def open_entries(exp, twins, field, batch):
    """Entries of target `field` of batch number `batch` that the twins move by more than a third of
    the tolerance (None if the batch has no such field)."""
    def pick(d):
        if field == "beliefs":
            x = d[batch]["features"]["beliefs"]
            return x.reshape(x.shape[0], 2, H)
        return d[batch].get(field)
    base = pick(exp)
    if base is None:
        return None
    tol = (TARGET_ATOL[field] + 1e-5 * np.abs(base)) / 3.0
    mask = np.zeros(base.shape, dtype=bool)
    for tw in twins:
        mask |= np.abs(pick(tw) - base) > tol
    return mask


WORST = {}


def close(got, exp, compared, open_, field, what):
    """`got` against `exp` on the entries of `compared` that are not `open_`."""
    m = np.broadcast_to(compared, got.shape) & ~np.broadcast_to(open_, got.shape)
    tol = TARGET_ATOL[field] + 1e-5 * np.abs(exp)
    ratio = np.where(m, np.abs(got - exp) / tol, 0.0)
    exempt = float(np.broadcast_to(open_, got.shape)[np.broadcast_to(compared, got.shape)].mean()) if got.size else 0.0
    worst = float(ratio.max()) if ratio.size else 0.0
    WORST[what] = max(WORST.get(what, 0.0), worst)
    assert worst <= TARGET_FACTOR, f"{what}: {int((ratio > TARGET_FACTOR).sum())} of {int(m.sum())} determined " \
                                   f"entries beyond {TARGET_FACTOR:g} tolerances, worst {worst:.2f}; exempt share {exempt:.2e}"
    assert exempt <= TARGET_MAX_EXEMPT, f"{what}: {exempt:.2e} of the entries are exempt"


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("fixture", ["base", "fused"])
@pytest.mark.parametrize("name", ["streets_mixed", "preflop", "linear_avg_zero_sum", "production_like"])
def test_training_data_matches_vectors_from_the_reference(golden_dir, name, fused, fixture):
    """``fixture`` "base": written by the reference's SparseCFREvaluator, compared on the hands the
    board allows (the product follows the fused class, which differs from the base class on
    blocked hands only); "fused": written by its FusedSparseCFREvaluator (Triton kernels under
    Triton's CPU interpreter), compared on every entry."""
    case, cols = load_case(golden_dir, name, fixture)
    if fixture == "base" and linear_plus(case):
        pytest.skip("the base class plays another strategy here (CFR+ clamp under linear CFR)")
    ev, r = golden_evaluator(case, fused)
    assert list(ev.depth_offsets) == case["depth_offsets"].tolist()
    n = ev.root_nodes
    assert np.array_equal(ev.env.last_board_indices[:n].cpu().numpy(), r["last_board_indices"])
    # the encoder alone on every node, board chosen by the leaf rule
    f = ev.feature_encoder.encode(ev.beliefs, pre_chance_node=ev.new_street_mask)
    np.testing.assert_allclose(f.context.cpu().numpy(), case["encode_leaf/context"], rtol=1e-6, atol=0)
    assert np.array_equal(f.board.cpu().numpy(), case["encode_leaf/board"])
    assert np.array_equal(f.to_act.cpu().numpy(), case["encode_leaf/to_act"])
    assert np.array_equal(f.street.cpu().numpy(), case["encode_leaf/street"])
    allowed_root = OC.allowed_hands_for_boards(r["board_indices"])[0]              # [n, H]
    if fixture == "fused":
        allowed_root = np.ones_like(allowed_root)
    batches = [batch_as_dict(b) for b in ev.training_data()]
    exp_o, twins_o = oracle_with_twins(case, ev, r, fused_variant=fixture == "fused")
    for bi, (got, tag) in enumerate(zip(batches, ("value", "pre_value", "policy"))):
        k = int(case[f"{tag}/len"])
        ft = got["features"]
        assert ft["context"].shape[0] == k
        if k == 0:
            continue
        np.testing.assert_allclose(ft["context"], case[f"{tag}/context"], rtol=1e-6, atol=0)
        assert np.array_equal(ft["board"], case[f"{tag}/board"])
        assert np.array_equal(ft["to_act"], case[f"{tag}/to_act"])
        assert np.array_equal(ft["street"], case[f"{tag}/street"])
        assert np.array_equal(got["legal_masks"], case[f"{tag}/legal_masks"])
        for s, v in got["statistics"].items():
            ref = case[f"{tag}/stat/{s}"]
            if np.issubdtype(ref.dtype, np.floating):
                np.testing.assert_allclose(v, ref, rtol=3e-3, atol=5e-5, err_msg=s)
            else:
                assert np.array_equal(v, ref), s
        # rows of this batch -> their roots, for the mask of hands the board allows
        if tag == "policy":
            rows = np.nonzero(~ev.tree.leaf_mask[:ev.depth_offsets[-2]])[0]
            root_of = ev.tree.root_index[rows]
        elif tag == "value":
            root_of = np.nonzero(~((r["street"] == 0) & (r["actions_this_round"] == 0)))[0]
        else:
            root_of = np.nonzero((r["actions_this_round"] == 0) & (r["street"] >= 1) & (r["street"] <= 3))[0]
        ok = allowed_root[root_of]                                                   # [k, H]
        fb = ft["beliefs"].reshape(k, 2, H)
        if tag == "pre_value":      # ranges before the deal: the hands the dealt cards block still carry mass
            np.testing.assert_allclose(fb[..., cols], case[f"{tag}/beliefs"], rtol=1e-6, atol=0)
        else:
            close(fb[..., cols], case[f"{tag}/beliefs"], ok[:, None, cols],
                  open_entries(exp_o, twins_o, "beliefs", bi)[..., cols], "beliefs", f"{tag} beliefs")
        if "value_targets" in got:
            mask = ok[:, None, :] if tag == "value" else np.ones((k, 1, H), bool)
            close(got["value_targets"], case[f"{tag}/value_targets"], mask,
                  open_entries(exp_o, twins_o, "value_targets", bi), "value_targets", f"{tag} value targets")
        if "policy_targets" in got:
            pt = got["policy_targets"]
            assert pt.shape == (k, H, len(BINS) + 3)
            close(pt[:, cols, :], case[f"{tag}/policy_targets"], ok[:, cols, None],
                  open_entries(exp_o, twins_o, "policy_targets", bi)[:, cols, :], "policy_targets", "policy targets")
            illegal = ~case[f"{tag}/legal_masks"]
            assert not pt.transpose(0, 2, 1)[illegal].any()                          # no child, no probability
    print(name, fixture, "worst determined entry, in tolerances:", {k: round(v, 2) for k, v in WORST.items()})


@pytest.mark.parametrize("name", ["streets_mixed", "linear_avg_zero_sum_warm", "production_like"])
def test_training_data_matches_oracle_everywhere(golden_dir, name):
    """Against the oracle following the one-kernel evaluator's conventions: every entry, blocked
    hands included.  The second case (linear CFR with CFR+, cfr_avg, zero-sum network, warm start)
    has no fused-class fixture — the reference's fused class cannot run its warm start there — so
    this comparison, with the oracle's base variant pinned on the same case, is what holds it."""
    case, _ = load_case(golden_dir, name)
    ev, r = golden_evaluator(case, True)
    exp, twins = oracle_with_twins(case, ev, r)
    got = [batch_as_dict(b) for b in ev.training_data()]

    def same(a, b, tw, path):
        if isinstance(b, dict):
            assert set(a) == set(b), path
            for k in b:
                same(a[k], b[k], [t[k] for t in tw], f"{path}/{k}")
        elif np.issubdtype(np.asarray(b).dtype, np.floating):
            leaf = path.rsplit("/", 1)[-1]
            if "local_" in path:                       # scalars out of the best-response pass
                np.testing.assert_allclose(a, b, rtol=3e-3, atol=5e-5, err_msg=path)
            elif leaf in TARGET_ATOL:
                tol = (TARGET_ATOL[leaf] + 1e-5 * np.abs(b)) / 3.0
                open_ = np.zeros(np.shape(b), dtype=bool)
                for t in tw:
                    open_ |= np.abs(t - b) > tol
                close(a, b, np.ones(np.shape(b), dtype=bool), open_, leaf, path)
            else:                                      # context features: the same float32 operations
                np.testing.assert_allclose(a, b, rtol=1e-6, atol=0, err_msg=path)
        else:
            assert np.array_equal(a, b), path
    for bi, (a, b, tag) in enumerate(zip(got, exp, ("value", "pre_value", "policy"))):
        same(a, b, [t[bi] for t in twins], tag)
    print(name, "worst determined entry, in tolerances:", {k: round(v, 2) for k, v in WORST.items()})


def test_policy_targets_kernel_matches_pull_back_on_a_deep_tree():
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.tree import RootStates
    from oracle import best_response as OBR
    from tests.helpers import random_boards
    rng = np.random.default_rng(43)
    n = 5
    boards = random_boards(rng, n, 5)
    roots = RootStates.at_round_start(3, rng.integers(100, 400, n), rng.integers(300, 2000, (n, 2)), boards)
    ev = HipSparseCFREvaluator(None, torch.device(DEV), river_dcfr_config(n, iterations=2, depth=5))
    ev.initialize_subgame(roots, np.arange(n))
    ev.policy_probs_avg.copy_(torch.from_numpy(rng.random((ev.total_nodes, H)).astype(np.float32)))
    top = ev.depth_offsets[-2]
    shim = SimpleNamespace(num_actions=ev.num_actions, parent_index=ev.tree.parent_index,
                           action_from_parent=ev.tree.action_from_parent,
                           _level=lambda level: (0, top, ev.depth_offsets[1], ev.total_nodes))
    exp = np.transpose(OBR.pull_back(shim, ev.policy_probs_avg.cpu().numpy()), (0, 2, 1))
    rows = torch.from_numpy(rng.permutation(top)[: top // 2]).to(DEV)             # any rows, any order, leaves too
    got = ev._policy_targets(rows).cpu().numpy()
    assert np.array_equal(got, exp[rows.cpu().numpy()])                             # a gather: exact
    # Childless rows of the last level: their child_offsets entry equals the row count, so a slot without
    # a child must request a row of the table itself (the node's own), never `child_offsets[r]`.
    last = torch.arange(ev.total_nodes - 3, ev.total_nodes, device=DEV)
    assert int(ev.child_count[last].sum()) == 0 and int(ev.child_offsets[last].max()) >= ev.total_nodes - 1
    assert not bool(ev._policy_targets(last).any())
    # the same into a buffer that is only 8-byte aligned (rows as float2 instead of whole 128-byte lines),
    # with guard floats on both sides
    from poker2_amd import _lib
    k, a = rows.numel(), ev.num_actions
    for offset in (0, 2):
        buf = torch.full((k * H * a + 8,), float("nan"), device=DEV)
        out = buf[offset:offset + k * H * a]
        _lib.call("p2hip_policy_targets", _lib.ptr(ev.policy_probs_avg), _lib.ptr(rows), k, _lib.ptr(ev.child_offsets),
                  _lib.ptr(ev.child_count), _lib.ptr(ev.action_from_parent), a, out.data_ptr(), _lib.stream_ptr())
        torch.cuda.synchronize()
        assert torch.isnan(buf[:offset]).all() and torch.isnan(buf[offset + k * H * a:]).all()
        assert np.array_equal(out.view(k, H, a).cpu().numpy(), got)
    assert ev._policy_targets(rows[:0]).shape == (0, H, ev.num_actions)
    with pytest.raises(IndexError):
        ev._policy_targets(torch.tensor([ev.total_nodes], device=DEV))


# ---- the loop around the search ---------------------------------------------------------------
class ListBuffer:
    def __init__(self):
        self.batches = []

    def add_batch(self, batch):
        self.batches.append(batch)


def test_sampled_leaves_are_dealt_from_the_runout_or_fresh_cards():
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.leaf_models import NetworkLeafModel
    from poker2_amd.tree import CARDS_ON_STREET, RootStates
    rng = np.random.default_rng(50)
    n = 64
    runout = np.stack([rng.permutation(52)[:5] for _ in range(n)]).astype(np.int64)
    boards = runout.copy()
    boards[:, 4] = -1                                                    # turn roots
    beliefs = torch.full((n, 2, H), 1.0 / H)
    for with_runout in (True, False):
        roots = RootStates.at_round_start(2, np.full(n, 200), np.tile([[900, 900]], (n, 1)), boards,
                                          button=np.arange(n) % 2)
        if with_runout:
            roots.runout = runout
        gen = torch.Generator(device=DEV)
        gen.manual_seed(5)
        ev = HipSparseCFREvaluator(NetworkLeafModel(ValueNet(), DEV), torch.device(DEV),
                                   river_dcfr_config(n, iterations=4, depth=3, dcfr_delay=0), generator=gen)
        ev.initialize_subgame(roots, np.arange(n), beliefs)
        nxt = ev.evaluate_cfr()
        k = nxt.nodes.numel()
        assert 0 < k <= n and nxt.env is nxt.roots and nxt.beliefs.shape == (k, 2, H)
        rows = nxt.nodes.cpu().numpy()
        root_of = ev.tree.root_index[rows]
        r = nxt.roots
        closed = ev.tree.new_street_mask[rows]
        assert closed.any() and (~closed).any()
        assert np.array_equal(r.street, np.where(closed, 3, 2))
        assert np.array_equal(r.last_board, boards[root_of])              # the board before any deal
        assert np.array_equal(r.board[:, :4], boards[root_of][:, :4])
        assert (r.board[~closed, 4] == -1).all()
        river = r.board[closed, 4]
        assert ((river >= 0) & (river < 52)).all()
        assert not (river[:, None] == boards[root_of][closed][:, :4]).any()   # a card that was not out yet
        if with_runout:
            assert np.array_equal(river, runout[root_of][closed, 4])
            assert np.array_equal(r.runout, runout[root_of])
        shown = np.arange(5)[None, :] < CARDS_ON_STREET[r.street][:, None]
        assert np.array_equal(np.where(shown, r.runout, -1), r.board)
        # the sampled states are valid roots of the next search, ranges included
        ev.initialize_subgame(r, np.arange(k), nxt.beliefs)
        ev.prepare_search()
        assert torch.isfinite(ev.values_avg).all()
        on_board = torch.zeros(k, 52, dtype=torch.bool)
        bb = torch.from_numpy(r.board)
        on_board[torch.arange(k)[:, None].expand(-1, 5)[bb >= 0], bb[bb >= 0]] = True
        from poker2_amd.card_utils import hand_combos_tensor
        cm = hand_combos_tensor()
        blocked = on_board[:, cm[:, 0]] | on_board[:, cm[:, 1]]
        assert not ev.beliefs[:k].cpu()[blocked[:, None, :].expand(-1, 2, -1)].any()   # the new card blocks hands


def test_data_generator_loop_plays_hands_forward():
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.leaf_models import NetworkLeafModel
    from poker2_amd.rebel_data_generator import EnvProto, RebelDataGenerator
    n = 24
    gen = torch.Generator(device=DEV)
    gen.manual_seed(11)
    cpu_gen = torch.Generator(device="cpu")
    cpu_gen.manual_seed(12)
    ev = HipSparseCFREvaluator(NetworkLeafModel(ValueNet(), DEV), torch.device(DEV),
                               river_dcfr_config(n, iterations=4, depth=3, dcfr_delay=0), generator=gen)
    ev.sample_epsilon = 0.25
    values, policies = ListBuffer(), ListBuffer()
    dg = RebelDataGenerator(EnvProto(mean_stack=1000, randomize_stacks=True, rng=cpu_gen), ev, values, policies)
    dg.evaluator.chance_helper.FLOP_SAMPLE_SIZE = 32            # keep the flop chance node small here
    assert dg.current_pbs.env.n == n and (dg.current_pbs.env.street == 0).all()
    streets_seen = set()
    total_value = 0
    for _ in range(4):
        value_batch, policy_batch = dg.generate_data(40)
        assert value_batch is not None and policy_batch is not None
        total_value += len(value_batch)
        streets_seen |= set(value_batch.statistics["street"].cpu().tolist())
        assert value_batch.value_targets.shape[1:] == (2, H) and policy_batch.policy_targets.shape[1:] == (H, 5)
        assert torch.isfinite(value_batch.value_targets).all() and value_batch.value_targets.abs().max() <= 1.0
        # a policy target row is a distribution over the legal actions for every hand the board allows
        s = policy_batch.policy_targets.sum(dim=2)
        assert ((s - 1.0).abs() < 1e-4).logical_or(s.abs() < 1e-6).all()
        assert not policy_batch.policy_targets.permute(0, 2, 1)[~policy_batch.legal_masks].any()
        assert dg.last_extra >= 0
        pbs = dg.current_pbs
        assert pbs.beliefs.shape[0] == pbs.env.n <= n
    assert len(values.batches) == 2 * len(policies.batches) and total_value >= 160
    assert {1, 2}.issubset(streets_seen)                         # hands move on to later streets
    # pre-chance samples: the state before the deal, on the previous street's board and stage
    pre = [b for b in values.batches[1::2] if len(b)]
    assert pre
    for b in pre:
        st = b.statistics["street"]
        assert (b.statistics["stage"] == 2 * st + 1).all()
        cards = (b.features.board >= 0).sum(dim=1).cpu()
        assert torch.equal(cards, torch.tensor([0, 3, 4, 5])[st.cpu()])


def test_leaf_model_does_not_reuse_features_of_the_previous_subgame():
    """Two subgames of identical shape on one evaluator: the second must see its own pots and boards."""
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.leaf_models import ChanceLeafModel, NetworkLeafModel, RangeBoardMLP
    from poker2_amd.tree import RootStates
    n = 8
    beliefs = torch.full((n, 2, H), 1.0 / H)

    def roots_of(pot, seed):
        r = np.random.default_rng(seed)
        boards = np.full((n, 5), -1, dtype=np.int64)
        boards[:, :4] = np.stack([r.permutation(52)[:4] for _ in range(n)])
        return RootStates.at_round_start(2, np.full(n, pot), np.tile([[900, 900]], (n, 1)), boards)
    first, second = roots_of(200, 1), roots_of(600, 2)
    net = RangeBoardMLP(hidden=32, layers=1, seed=1).to(DEV)
    for make in (lambda: NetworkLeafModel(ValueNet(), DEV), lambda: ChanceLeafModel(net, DEV)):
        cfg = river_dcfr_config(n, iterations=2, depth=2, dcfr_delay=0)
        ev = HipSparseCFREvaluator(make(), torch.device(DEV), cfg, max_raises=1)
        ev.initialize_subgame(first, np.arange(n), beliefs)
        ev.prepare_search()
        ev.initialize_subgame(second, np.arange(n), beliefs)
        ev.prepare_search()
        fresh = HipSparseCFREvaluator(make(), torch.device(DEV), cfg, max_raises=1)
        fresh.initialize_subgame(second, np.arange(n), beliefs)
        fresh.prepare_search()
        assert torch.equal(ev.model_indices, fresh.model_indices)
        assert torch.equal(ev.latest_values, fresh.latest_values)
        assert ev.latest_values[ev.model_indices].abs().max() > 0


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("fixture", ["base", "fused"])
@pytest.mark.parametrize("name", ["streets_mixed", "preflop", "linear_avg_zero_sum", "production_like"])
def test_whole_search_from_a_seeded_generator_samples_the_reference_leaves(golden_dir, name, fused, fixture):
    """``evaluate_cfr`` with its random parts — the sampling schedule, the hand and exploration
    draws of the leaf walk (cfr_evaluator.py:1497-1528, :382-404, sparse_cfr_evaluator.py:325-426)
    — from a CPU generator with the seed the reference run used: the same iterations are
    snapshotted, the same leaves come out, and leaves that closed a betting round stand on the
    next street with the cards the env's deck deals."""
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.leaf_models import NetworkLeafModel
    from poker2_amd.tree import RootStates
    case, cols = load_case(golden_dir, name, fixture)
    r = {k[5:]: v for k, v in case.items() if k.startswith("root/")}
    n = len(r["street"])
    roots = RootStates.from_env(SimpleNamespace(bb=100, deck=case["search/root_deck"], **r), np.arange(n))
    assert np.array_equal(roots.runout, case["search/root_deck"][:, 4:9])
    depth, iters, algo = case_settings(case)
    if fixture == "base" and linear_plus(case):
        pytest.skip("the base class plays another strategy here (CFR+ clamp under linear CFR)")
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(case["search/seed"]))
    ev = HipSparseCFREvaluator(NetworkLeafModel(ValueNet(), DEV, enforce_zero_sum=algo["enforce_zero_sum"]),
                               torch.device(DEV), search_config(n, depth, iters, algo), generator=gen,
                               fused_iteration=fused)
    ev.initialize_subgame(roots, np.arange(n), torch.from_numpy(case["beliefs"]))
    leaves = ev.evaluate_cfr(training_mode=True)
    assert np.array_equal(ev.t_sample.cpu().numpy(), case["search/t_sample"])
    got = leaves.roots
    names = {"board": "board_indices", "last_board": "last_board_indices"}
    for field in ("street", "to_act", "button", "pot", "stacks", "committed", "min_raise", "actions_this_round",
                  "is_allin", "starting_stacks", "scale", "board", "last_board", "done"):
        want = case[f"search/leaf/{names.get(field, field)}"]
        assert np.array_equal(np.asarray(getattr(got, field)), want.astype(np.asarray(getattr(got, field)).dtype)), field
    assert np.array_equal(got.runout, case["search/leaf/deck"][:, 4:9])          # the deck travels with the state
    lb = leaves.beliefs.cpu().numpy()
    np.testing.assert_allclose(lb[..., cols], case["search/leaf_beliefs"], rtol=3e-4, atol=3e-6)
    np.testing.assert_allclose(lb.sum(-1, dtype=np.float64), case["search/leaf_beliefs_rowsum"], rtol=1e-4)


def compare_generator_batch(g, prefix, batch, cols, every_entry):
    """One batch the loop stored or returned against the fixture's.  ``every_entry``: the fixture
    comes from the reference's fused class, whose conventions on board-blocked hands the product
    shares; otherwise hands that the batch's own board blocks are left out of the float checks."""
    n = int(g[f"{prefix}/len"])
    assert len(batch) == n, prefix
    if n == 0:
        return
    f = batch.features
    np.testing.assert_allclose(f.context.cpu().numpy(), g[f"{prefix}/context"], rtol=1e-6, atol=0, err_msg=prefix)
    board = f.board.cpu().numpy()
    assert np.array_equal(board, g[f"{prefix}/board"]), prefix
    assert np.array_equal(f.to_act.cpu().numpy(), g[f"{prefix}/to_act"]), prefix
    assert np.array_equal(f.street.cpu().numpy(), g[f"{prefix}/street"]), prefix
    assert np.array_equal(batch.legal_masks.cpu().numpy(), g[f"{prefix}/legal_masks"]), prefix
    ok = np.ones((n, H), bool) if every_entry else OC.allowed_hands_for_boards(board)[0]
    # No oracle runs this loop, so there are no twins to say which entries are open: every compared entry
    # is held, without exemption, to LOOP_FACTOR x (1e-5 relative + TARGET_ATOL) — three iterations of
    # regret matching per search, nine searches feeding one another (measured; the numerics of one
    # search are what the tests above hold tightly).
    def all_close(got, exp, compared, field, what):
        m = np.broadcast_to(compared, got.shape)
        ratio = np.where(m, np.abs(got - exp) / (TARGET_ATOL[field] + 1e-5 * np.abs(exp)), 0.0)
        WORST[what.split("/")[-1]] = max(WORST.get(what.split("/")[-1], 0.0), float(ratio.max()))
        assert ratio.max() <= LOOP_FACTOR, f"{what}: worst entry {ratio.max():.1f} tolerances (bound {LOOP_FACTOR:g})"
    fb = f.beliefs.cpu().numpy().reshape(n, 2, H)
    all_close(fb[..., cols], g[f"{prefix}/beliefs"], ok[:, None, cols], "beliefs", f"{prefix} beliefs")
    if batch.value_targets is not None:
        vt = batch.value_targets.cpu().numpy()
        all_close(vt[..., cols], g[f"{prefix}/value_targets"], ok[:, None, cols], "value_targets", f"{prefix} value targets")
    if batch.policy_targets is not None:
        pt = batch.policy_targets.cpu().numpy()
        all_close(pt[:, cols, :], g[f"{prefix}/policy_targets"], ok[:, cols, None], "policy_targets", f"{prefix} policy targets")


@pytest.mark.parametrize("reuse_state", [False, True])
@pytest.mark.parametrize("fixture", ["base", "fused"])
def test_generator_loop_reproduces_the_reference_run(golden_dir, fixture, reuse_state):
    """The whole self-play loop (rebel_data_generator.py:52-95) against a run of the reference's own
    generator, evaluator and env from the same two seeds: the same hands are dealt, the same
    batches reach the buffers pass by pass, the call returns the same samples and leaves the same
    public states behind — decks included, so the next call would deal the same cards."""
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.leaf_models import NetworkLeafModel
    from poker2_amd.rebel_data_generator import EnvProto, RebelDataGenerator
    g = np.load(str(golden_dir) + ("/fused_generator_golden.npz" if fixture == "fused" else "/generator_golden.npz"))
    n, depth, iters, asked, env_seed, search_seed = (int(x) for x in g["settings"])
    cols = g["columns"]
    WORST.clear()
    env_gen, search_gen = torch.Generator(device="cpu"), torch.Generator(device="cpu")
    env_gen.manual_seed(env_seed)
    search_gen.manual_seed(search_seed)
    proto = EnvProto(mean_stack=1000, sb=50, bb=100, randomize_stacks=True, rng=env_gen)
    ev = HipSparseCFREvaluator(NetworkLeafModel(ValueNet(), DEV), torch.device(DEV),
                               river_dcfr_config(n, iterations=iters, depth=depth, dcfr_delay=0), generator=search_gen,
                               reuse_state=reuse_state)         # the buffers keep every pass's batches: nothing may alias the state

    class Recorder:
        def __init__(self):
            self.batches = []

        def add_batch(self, batch):
            self.batches.append(batch)
    value_buffer, policy_buffer = Recorder(), Recorder()
    dg = RebelDataGenerator(proto, ev, value_buffer, policy_buffer)

    def same_states(tag, roots):
        names = {"board": "board_indices", "last_board": "last_board_indices"}
        for field in ("street", "to_act", "button", "pot", "stacks", "committed", "min_raise", "actions_this_round",
                      "is_allin", "starting_stacks", "scale", "board", "done"):
            got = np.asarray(getattr(roots, field))
            assert np.array_equal(got, g[f"{tag}/{names.get(field, field)}"].astype(got.dtype)), (tag, field)
        assert np.array_equal(roots.runout, g[f"{tag}/deck"][:, 4:9]), tag
        assert np.array_equal(roots.previous_board(), g[f"{tag}/last_board_indices"]), tag
    same_states("first_deal", dg.current_pbs.env)
    value_batch, policy_batch = dg.generate_data(asked)
    every = fixture == "fused"
    assert len(policy_buffer.batches) == int(g["passes"]) and len(value_buffer.batches) == 2 * int(g["passes"])
    for i, b in enumerate(value_buffer.batches):
        compare_generator_batch(g, f"value_buffer/{i}", b, cols, every or i % 2 == 1)   # odd adds: ranges before the deal
    for i, b in enumerate(policy_buffer.batches):
        compare_generator_batch(g, f"policy_buffer/{i}", b, cols, every)
    assert len(value_batch) == int(g["returned/value/len"]) and len(policy_batch) == int(g["returned/policy/len"])
    assert np.array_equal(value_batch.features.board.cpu().numpy(), g["returned/value/board"])
    assert np.array_equal(policy_batch.features.board.cpu().numpy(), g["returned/policy/board"])
    assert dg.last_extra == int(g["last_extra"])
    same_states("left", dg.current_pbs.env)
    lb = dg.current_pbs.beliefs.cpu().numpy()
    ok = np.ones(lb.shape[::2], bool) if every else OC.allowed_hands_for_boards(g["left/board_indices"])[0]
    ratio = np.where(ok[:, None, cols], np.abs(lb[..., cols] - g["left/beliefs"]) /
                     (TARGET_ATOL["beliefs"] + 1e-5 * np.abs(g["left/beliefs"])), 0.0)
    assert ratio.max() <= LOOP_FACTOR, f"beliefs left behind: worst entry {ratio.max():.1f} tolerances"
    print(fixture, "loop: worst entry, in tolerances:", {k: round(v, 1) for k, v in WORST.items()},
          "beliefs left behind", round(float(ratio.max()), 1))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_leaf_rows_to_the_network_and_back(dtype):
    """``gather_leaf_rows`` / the scatter behind ``set_leaf_values`` against the torch operations they
    replace (``table[rows]`` + ``.to(dtype)`` + ``cat``; ``.to(float32)`` + ``index_copy_``):
    bit-exact, conversions included (bfloat16 rounds to nearest even, NaN stays NaN), columns behind
    the ranges untouched, rows outside the table skipped."""
    from poker2_amd import _lib
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.tree import RootStates
    from tests.helpers import random_boards
    rng = np.random.default_rng(3)
    n = 6
    roots = RootStates.at_round_start(3, np.full(n, 200), np.tile([[800, 800]], (n, 1)), random_boards(rng, n, 5))
    ev = HipSparseCFREvaluator(None, torch.device(DEV), river_dcfr_config(n, iterations=2, depth=2))
    ev.initialize_subgame(roots, np.arange(n))
    total = ev.total_nodes
    table = torch.from_numpy(rng.standard_normal((total, 2, H)).astype(np.float32) * 3.0).to(DEV)
    table[1, 0, 5] = float("nan")
    table[2, 1, 7] = float("inf")
    table[3, 0, 9] = 1e-41                                   # denormal
    others = rng.permutation(np.arange(4, total))[:34]
    rows = torch.from_numpy(np.concatenate([[1, 2, 3], others]).astype(np.int64)).to(DEV)      # distinct rows
    width = 2 * H + 52
    out = torch.full((37, width), 7.0, dtype=dtype, device=DEV)
    ev.gather_leaf_rows(table, rows, out)
    want = table[rows].reshape(37, -1).to(dtype)
    assert torch.equal(out[:, :2 * H].view(torch.int16 if dtype != torch.float32 else torch.int32),
                       want.view(torch.int16 if dtype != torch.float32 else torch.int32))
    assert (out[:, 2 * H:] == 7.0).all()
    # and back
    answers = torch.from_numpy(rng.standard_normal((37, 2, H)).astype(np.float32)).to(DEV).to(dtype)
    dst = torch.full((total, 2, H), -5.0, device=DEV)
    bad = rows.clone()
    bad[4], bad[5] = -1, total                               # outside the table: skipped
    _lib.call("p2hip_scatter_leaf_rows", _lib.ptr(answers), {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}[dtype],
              2 * H, _lib.ptr(bad), 37, _lib.ptr(dst), total, _lib.stream_ptr())
    want = torch.full((total, 2, H), -5.0, device=DEV)
    keep = torch.ones(37, dtype=torch.bool, device=DEV)
    keep[4] = keep[5] = False
    want.index_copy_(0, rows[keep], answers[keep].float())
    assert torch.equal(dst, want)


def test_network_answers_do_not_depend_on_how_the_ranges_reach_it():
    """NetworkLeafModel over RangeBoardMLP: ranges written straight into the kept input matrix
    (``leaf_values_from_nodes``) against gather + concatenate + cast (``leaf_values``), float32 and
    bf16 autocast: identical answers, and identical searches."""
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.leaf_models import NetworkLeafModel, RangeBoardMLP
    from poker2_amd.tree import RootStates
    from tests.helpers import random_boards, random_ranges
    rng = np.random.default_rng(8)
    n = 5
    boards = random_boards(rng, n, 5)
    boards[:3, 4] = -1                                        # three turn roots: street-end leaves go to the network
    beliefs = torch.from_numpy(random_ranges(rng, boards))
    roots = RootStates.at_round_start(np.where(boards[:, 4] < 0, 2, 3), np.full(n, 200), np.tile([[800, 800]], (n, 1)), boards)
    net = RangeBoardMLP(hidden=64, layers=2, seed=2).to(DEV)
    for autocast in (None, torch.bfloat16):
        states = []
        for direct in (True, False):
            model = NetworkLeafModel(net, DEV, autocast_dtype=autocast)
            ev = HipSparseCFREvaluator(model if direct else _WithoutNodes(model), torch.device(DEV),
                                       river_dcfr_config(n, iterations=4, depth=16), max_raises=1)
            ev.initialize_subgame(roots, np.arange(n), beliefs)
            ev.prepare_search(t_sample=torch.full((ev.total_nodes,), -1, dtype=torch.long))
            assert ev.model_indices.numel() > 0
            for t in range(3):
                ev.cfr_iteration(t)
            states.append({k: getattr(ev, k).clone() for k in OCFR.OracleCFR.STATE_NAMES})
        for k in OCFR.OracleCFR.STATE_NAMES:
            assert torch.equal(states[0][k], states[1][k]), (autocast, k)


class _WithoutNodes:
    """A leaf model that only offers ``leaf_values`` (the evaluator then gathers the ranges itself)."""

    def __init__(self, inner):
        self.inner = inner
        self.enforce_zero_sum = inner.enforce_zero_sum

    def leaf_values(self, beliefs, rows, ev):
        return self.inner.leaf_values(beliefs, rows, ev)


def test_evaluator_takes_a_bare_network_like_the_reference():
    """``Evaluator(model, device, cfg)`` with the network itself, as the reference's trainer builds it
    (src/p2/rl/cfr_trainer.py:194-207): the constructor wraps it in NetworkLeafModel — same search as with
    the explicit wrapper, ``enforce_zero_sum`` read off the network (cfr_evaluator.py:970) — and a network
    with a policy head, called as the reference calls it (``model(features, include_policy=True)``,
    :305-329), sets the initial policy."""
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.leaf_models import NetworkLeafModel, RangeBoardMLP
    from poker2_amd.tree import RootStates
    from tests.helpers import random_boards, random_ranges
    rng = np.random.default_rng(18)
    n = 4
    boards = random_boards(rng, n, 5)
    boards[:2, 4] = -1
    beliefs = torch.from_numpy(random_ranges(rng, boards))
    roots = RootStates.at_round_start(np.where(boards[:, 4] < 0, 2, 3), np.full(n, 200), np.tile([[800, 800]], (n, 1)), boards)

    def search(model):
        ev = HipSparseCFREvaluator(model, torch.device(DEV), river_dcfr_config(n, iterations=4, depth=16), max_raises=1)
        ev.initialize_subgame(roots, np.arange(n), beliefs)
        ev.prepare_search(t_sample=torch.full((ev.total_nodes,), -1, dtype=torch.long))
        first_policy = ev.policy_probs.clone()
        ev.run_search_iterations()
        return ev, first_policy

    net = RangeBoardMLP(hidden=64, layers=2, seed=3).to(DEV)
    bare, _ = search(net)
    wrapped, _ = search(NetworkLeafModel(net, DEV))
    assert isinstance(bare.model, NetworkLeafModel) and bare.model.net is net and not bare.enforce_zero_sum
    assert bare.model_indices.numel() > 0
    for k in OCFR.OracleCFR.STATE_NAMES:
        assert torch.equal(getattr(bare, k), getattr(wrapped, k)), k

    class PolicyNet(torch.nn.Module):
        enforce_zero_sum = True

        def __init__(self, actions):
            super().__init__()
            self.actions = actions
            self.calls = []

        def forward(self, f, include_policy=True):
            self.calls.append(include_policy)
            k = f.beliefs.shape[0]
            hv = 0.01 * (f.beliefs.view(k, 2, H).flip(1) * H - 1.0)
            logits = None
            if include_policy:
                hand = torch.arange(H, device=f.beliefs.device, dtype=torch.float32)
                act = torch.arange(self.actions, device=f.beliefs.device, dtype=torch.float32)
                logits = torch.sin(0.01 * hand[None, :, None] * (1.0 + act[None, None, :])) + f.context[:, 1, None, None]
            return SimpleNamespace(hand_values=hv, policy_logits=logits)

    pnet = PolicyNet(5)
    ev, first_policy = search(pnet)
    assert ev.enforce_zero_sum and True in pnet.calls and False in pnet.calls
    # root level by hand: softmax over the legal actions of the network's logits, one child row per action
    hand = torch.arange(H, device=DEV, dtype=torch.float32)
    act = torch.arange(5, device=DEV, dtype=torch.float32)
    feats = ev.feature_encoder.encode(ev.beliefs, indices=torch.arange(n, device=DEV))
    logits = torch.sin(0.01 * hand[None, :, None] * (1.0 + act[None, None, :])) + feats.context[:, 1, None, None]
    probs = torch.softmax(logits.masked_fill(~ev.legal_mask[:n, None, :], float("-inf")), dim=-1)
    lo, hi = ev.depth_offsets[1], ev.depth_offsets[2]
    want = probs[ev.parent_index[lo:hi], :, ev.action_from_parent[lo:hi]]
    assert torch.allclose(first_policy[lo:hi], want, rtol=1e-6, atol=1e-7)
    assert float((first_policy[lo:hi] - 1.0 / ev.child_count[ev.parent_index[lo:hi]][:, None]).abs().max()) > 0.05
