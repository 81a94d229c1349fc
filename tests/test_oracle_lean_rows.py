"""CPU: which rows of the state an iteration may leave unwritten when nobody looks at the state before
the next iteration (the product's lean launches).  The oracle runs twice: as it is, and with the rows
the rule below calls dead overwritten by NaN after every iteration but the last.  If a single dead
entry were read by the next iteration, NaN would spread into the final state; the test demands the
eleven tensors of the two runs to be bit-identical.

The rule (restated here from the reads of one iteration, src/p2/search/fused_sparse_cfr_evaluator.py:478-533):
  * self_reach / self_reach_avg of a row are read only by the reach step of its own children
    (:153-172) and, for self_reach_avg, by the average-policy mix of its children (:355-398);
  * beliefs of a row are read by the regret weights and the value backup at rows with children
    (:312-349, :242-306) and by the leaf evaluations (showdown rows, rows sent to the leaf network, :447-472);
    under cfr_avg the regret weights and leaf evaluations read beliefs_avg instead (:322, :455);
  * beliefs_avg is otherwise read only by the zero-sum shift of the average values (:404-414), on every row.
"""
import numpy as np
import pytest

from oracle import cfr as OCFR
from tests.helpers import random_boards, random_ranges
from tests.test_oracle_cfr import river_tree

STATE = ("policy_probs", "policy_probs_avg", "policy_probs_sample", "cumulative_regrets", "regret_weight_sums",
         "self_reach", "self_reach_avg", "beliefs", "beliefs_avg", "latest_values", "values_avg")


def dead_rows(o: OCFR.OracleCFR, has_model: bool) -> dict:
    """name -> boolean row mask of the rows a lean iteration does not store."""
    n, total = o.root_nodes, o.total_nodes
    below_root = np.arange(total) >= n
    parent = o.child_count > 0
    leaf_eval = np.asarray(o.tree["showdown_mask"]) | ((o.leaf_mask & ~o.done) if has_model else False)
    keep_b = parent | (leaf_eval & (not o.cfr_avg))
    if o.enforce_zero_sum:
        keep_ba = np.ones(total, bool)
    elif o.cfr_avg:
        keep_ba = parent | leaf_eval
    else:
        keep_ba = np.zeros(total, bool)
    return {"self_reach": below_root & ~parent, "self_reach_avg": below_root & ~parent,
            "beliefs": below_root & ~keep_b, "beliefs_avg": below_root & ~keep_ba}


CASES = {
    "discounted": dict(cfr_type="discounted"),
    "discounted_delay": dict(cfr_type="discounted", dcfr_delay=3),
    "discounted_plus_cfrplus": dict(cfr_type="discounted_plus", dcfr_delay=2, cfr_plus=True),
    "linear_cfr_avg": dict(cfr_type="linear", cfr_avg=True, cfr_plus=True),
    "standard_zero_sum": dict(cfr_type="standard", enforce_zero_sum=True),
    "linear_cfr_avg_zero_sum_model": dict(cfr_type="linear", cfr_avg=True, enforce_zero_sum=True, model=True),
    "discounted_model": dict(cfr_type="discounted", model=True),
    "final_policy_values": dict(cfr_type="discounted", use_final_policy_values=True),
}


@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("fused_variant", [False, True])
def test_rows_a_lean_iteration_skips_are_never_read(name, fused_variant):
    kw = dict(CASES[name])
    has_model = kw.pop("model", False)
    rng = np.random.default_rng(11)
    n, iters = 2, 7
    t = river_tree(n, depth=3)
    boards = random_boards(rng, n)
    bel = random_ranges(rng, boards)

    def leaf_values(beliefs, rows):
        # a network stand-in that depends on the ranges it is shown (rows of the leaves only)
        b = beliefs[rows]
        return (0.3 * (b[:, ::-1] * 1326.0 - 1.0).clip(-1, 1) * np.linspace(-1, 1, 1326, dtype=np.float32)).astype(np.float32)

    def run(poison: bool):
        o = OCFR.OracleCFR(t, boards, bel, cfr_iterations=iters, fused_variant=fused_variant,
                           t_sample_roots=np.array([2, 4]), leaf_value_fn=leaf_values if has_model else None, **kw)
        o.prepare()
        dead = dead_rows(o, has_model)
        assert all(m.any() for k, m in dead.items() if k != "beliefs_avg" or not o.enforce_zero_sum)
        for it in range(iters):
            o.cfr_iteration(it)
            if poison and it + 1 < iters:
                for k, m in dead.items():
                    getattr(o, k)[m] = np.nan
        return {k: getattr(o, k).copy() for k in STATE}

    a, b = run(False), run(True)
    for k in STATE:
        assert np.isfinite(b[k]).all(), k
        assert np.array_equal(a[k], b[k]), k
