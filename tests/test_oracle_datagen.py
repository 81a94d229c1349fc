"""CPU: pins the oracle's restatement of feature encoding and training targets
(src/p2/models/mlp/rebel_feature_encoder.py:55-127, src/p2/search/cfr_evaluator.py:1383-1495)
against vectors written by running the reference's evaluator (tests/golden/gen_training_data_golden.py)."""
import numpy as np
import pytest

from oracle import cfr as OCFR
from oracle import chance as OCH
from oracle import datagen as ODG
from oracle import tree as OT

H = 1326
BINS = [0.5, 1.0]


def value_net_numpy(context, street, to_act, board, beliefs):
    """numpy twin of ``ValueNet`` in tests/golden/gen_training_data_golden.py."""
    f32 = np.float32
    b = beliefs.reshape(-1, 2, H).astype(f32)
    ranks = np.where(board >= 0, (board % 13 + 1).astype(f32), f32(0.0))
    w = (f32(0.2) + f32(0.1) * context[:, 2] + f32(0.05) * context[:, 1] - f32(0.03) * context[:, 3]
         + f32(0.01 / 13.0) * ranks.sum(axis=1, dtype=f32)).astype(f32)
    opp = b[:, ::-1, :]
    sign = np.array([1.0, -1.0], f32)[None, :, None]
    h = ((np.arange(H) % 7).astype(f32) - f32(3.0)) * f32(0.002)
    return (sign * f32(0.05) * w[:, None, None] * (f32(H) * opp - f32(1.0)) + h[None, None, :]).astype(f32)


def load_case(golden_dir, name, fixture="base"):
    """``fixture``: "base" = written by the reference's SparseCFREvaluator, "fused" = by its
    FusedSparseCFREvaluator with the Triton kernels under Triton's CPU interpreter."""
    g = np.load(str(golden_dir) + ("/fused_training_data_golden.npz" if fixture == "fused" else
                                   "/training_data_golden.npz"))
    return {k[len(name) + 1:]: g[k] for k in g.files if k.startswith(name + "/")}, g["columns"]


CASE_NAMES = ["streets_mixed", "preflop", "linear_avg_zero_sum", "linear_avg_zero_sum_warm", "production_like"]
BASE_ONLY = {"linear_avg_zero_sum_warm"}      # the reference's fused class runs its warm start on unfilled scalars


def case_settings(case):
    """(depth, last iteration + 1, search settings) of a fixture case."""
    import json
    st = [str(x) for x in case["settings"]]
    return int(st[0]), int(st[1]), json.loads(st[2])


def oracle_search_arguments(algo):
    return dict(cfr_type=algo["cfr_type"], cfr_plus=algo["cfr_plus"], cfr_avg=algo["cfr_avg"],
                warm_start_iterations=algo["warm"], warm_start_type=algo["warm_type"],
                warm_start_multiplier=algo["warm_mult"], enforce_zero_sum=algo["enforce_zero_sum"],
                dcfr_delay=algo["delay"], dcfr_alpha=algo["alpha"], dcfr_beta=algo["beta"], dcfr_gamma=algo["gamma"],
                dcfr_alpha_final=algo["alpha_final"], dcfr_beta_final=algo["beta_final"],
                dcfr_gamma_final=algo["gamma_final"], use_final_policy_values=algo["final_policy_values"])


def oracle_roots(case):
    r = {k[5:]: v for k, v in case.items() if k.startswith("root/")}
    return [OT.Node(to_act=int(r["to_act"][i]), button=int(r["button"][i]), street=int(r["street"][i]),
                    pot=int(r["pot"][i]), stacks=r["stacks"][i].tolist(), committed=r["committed"][i].tolist(),
                    min_raise=int(r["min_raise"][i]), actions_this_round=int(r["actions_this_round"][i]),
                    is_allin=r["is_allin"][i].tolist(), starting_stacks=r["starting_stacks"][i].tolist(),
                    scale=float(r["scale"][i])) for i in range(len(r["street"]))], r


def run_oracle(case, fused_variant=False):
    roots, r = oracle_roots(case)
    depth, iters, algo = case_settings(case)
    tree = OT.build_tree(roots, BINS, depth)
    env = ODG.tree_env(tree, r["board_indices"])
    assert np.array_equal(env["last_board_indices"][:len(roots)], r["last_board_indices"])   # the derived rule

    def leaf_fn(beliefs, rows):
        f = ODG.encode(env, beliefs, pre_chance_node=tree["new_street_mask"], indices=rows)
        return value_net_numpy(f["context"], f["street"], f["to_act"], f["board"], f["beliefs"])
    o = OCFR.OracleCFR(tree, r["board_indices"], case["beliefs"], cfr_iterations=iters, leaf_value_fn=leaf_fn,
                       t_sample_roots=np.full(len(roots), -1, dtype=np.int64), fused_variant=fused_variant,
                       **oracle_search_arguments(algo))
    o.prepare()                                   # includes the warm start
    for t in range(algo["warm"], iters):
        o.cfr_iteration(t)
    if o.use_final_policy_values:
        o.update_average_values_final()
    return o, tree, env


def assert_close_but_few(got, exp, rtol, atol, what, frac=5e-4, cap=1e-4):
    """All entries within tolerance, except at most max(2, ``frac`` of them) that sit where regret
    matching divides by a small sum; none of those off by more than ``cap``."""
    diff = np.abs(np.asarray(got, dtype=np.float64) - exp)
    over = diff > atol + rtol * np.abs(exp)
    assert over.sum() <= max(2, frac * diff.size) and (not over.any() or diff[over].max() < cap), \
        f"{what}: {int(over.sum())} of {diff.size} entries over tolerance, max abs diff {diff.max():.3e}"


def check_batch(got, case, tag, cols, rtol, atol):
    n = int(case[f"{tag}/len"])
    f = got["features"]
    assert f["context"].shape[0] == n
    if n == 0:
        return
    np.testing.assert_allclose(f["context"], case[f"{tag}/context"], rtol=1e-6, atol=0)
    assert np.array_equal(f["board"], case[f"{tag}/board"])
    assert np.array_equal(f["to_act"], case[f"{tag}/to_act"])
    assert np.array_equal(f["street"], case[f"{tag}/street"])
    fb = f["beliefs"].reshape(n, 2, H)
    np.testing.assert_allclose(fb[..., cols], case[f"{tag}/beliefs"], rtol=rtol, atol=atol)
    np.testing.assert_allclose(fb.sum(-1, dtype=np.float64), case[f"{tag}/beliefs_rowsum"], rtol=rtol)
    assert np.array_equal(got["legal_masks"], case[f"{tag}/legal_masks"])
    if "value_targets" in got:
        np.testing.assert_allclose(got["value_targets"], case[f"{tag}/value_targets"], rtol=rtol, atol=atol)
    if "policy_targets" in got:
        pt = got["policy_targets"]
        assert pt.shape == (n, H, len(BINS) + 3)
        assert_close_but_few(pt[:, cols, :], case[f"{tag}/policy_targets"], rtol, atol, "policy targets")
        np.testing.assert_allclose(pt.sum(axis=1, dtype=np.float64), case[f"{tag}/policy_targets_sum"], rtol=rtol,
                                   atol=atol)
    for k, v in got["statistics"].items():
        ref = case[f"{tag}/stat/{k}"]
        if np.issubdtype(ref.dtype, np.floating):
            np.testing.assert_allclose(v, ref, rtol=2e-3, atol=2e-5, err_msg=k)   # sums of ~1e3 float32 products
        else:
            assert np.array_equal(v, ref), k


@pytest.mark.parametrize("fixture", ["base", "fused"])
@pytest.mark.parametrize("name", CASE_NAMES)
def test_oracle_training_data_matches_vectors_from_the_reference(golden_dir, name, fixture):
    if fixture == "fused" and name in BASE_ONLY:
        pytest.skip("no fused-class fixture for this case")
    case, cols = load_case(golden_dir, name, fixture)
    o, tree, env = run_oracle(case, fused_variant=fixture == "fused")
    assert o.depth_offsets == case["depth_offsets"].tolist()
    assert np.array_equal(tree["new_street_mask"], case["new_street_mask"])
    assert np.array_equal(tree["leaf_mask"], case["leaf_mask"])
    # the encoder alone on every node, board chosen by the leaf rule
    f = ODG.encode(env, o.beliefs, pre_chance_node=tree["new_street_mask"])
    np.testing.assert_allclose(f["context"], case["encode_leaf/context"], rtol=1e-6, atol=0)
    assert np.array_equal(f["board"], case["encode_leaf/board"])
    assert np.array_equal(f["to_act"], case["encode_leaf/to_act"])
    assert np.array_equal(f["street"], case["encode_leaf/street"])
    # the search state the targets come from (float32 1e-5 relative; 4 iterations)
    for s in ("policy_probs_avg", "beliefs", "beliefs_avg", "values_avg"):
        x = getattr(o, s)
        # values are sums of products with quotients of unblocked masses (showdown denominators, opponent
        # weights): on hands that face little compatible mass a 1e-7 in a range moves them by 1e-4
        wide = dict(frac=2e-3, cap=1e-3) if s == "values_avg" else {}
        assert_close_but_few(x[..., cols], case[f"state/{s}"], 2e-4, 2e-6, s, **wide)
    flop_tables = None
    if ((case["root/street"] == 1) & (case["root/actions_this_round"] == 0)).any():
        canonical, count, _ = OCH.canonical_flops()
        flop_tables = (canonical, count, OCH.combo_suit_perms())
    batches = ODG.training_data(o, env, BINS, value_net_numpy, flop_tables=flop_tables)
    for got, tag in zip(batches, ("value", "pre_value", "policy")):
        check_batch(got, case, tag, cols, rtol=2e-4, atol=2e-6)


def test_encode_closed_forms():
    env = {"to_act": np.array([0, 1, 0]), "button": np.array([1, 1, 0]),
           "starting_stacks": np.array([[1000, 1000], [0, 0], [10, 10]]), "pot": np.array([500, 7, 4000]),
           "committed": np.array([[0, 0], [100, 0], [100, 0]]), "actions_this_round": np.array([3, 0, 2]),
           "board_indices": np.arange(15).reshape(3, 5), "last_board_indices": -np.ones((3, 5), np.int64)}
    bel = np.zeros((3, 2, H), np.float32)
    f = ODG.encode(env, bel, pre_chance_node=np.array([False, True, False]))
    # (to_act - button) mod 2 is never negative; pot fraction clamps at 10 and guards a zero total;
    # the bet flag needs unequal chips AND an action this round
    assert f["context"].tolist() == [[0.0, 1.0, 0.25, 0.0], [1.0, 0.0, 7.0, 0.0], [0.0, 0.0, 10.0, 1.0]]
    assert f["board"].tolist() == [[0, 1, 2, 3, 4], [-1] * 5, [10, 11, 12, 13, 14]]
    assert f["beliefs"].shape == (3, 2 * H)
    sel = ODG.encode(env, bel, pre_chance_node=True, indices=np.array([2, 0]))
    assert sel["context"][:, 2].tolist() == [10.0, 0.25] and (sel["board"] == -1).all()
