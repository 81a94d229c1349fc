"""CPU: the numpy restatement of the per-operation CFR kernels (oracle/cfr_ops.py,
oracle/unblocked.py) against outputs of the reference's own Triton kernels, run under Triton's
CPU interpreter by tests/golden/gen_fused_ops_golden.py.  Inputs are rebuilt from the same seeds.

Tolerance: 1e-5 relative (+1e-6 absolute) per element, the bound the path states for fp32; row
sums (float64 sums of fp32 outputs) to 1e-5 of the row's absolute mass plus a fifth of the
per-element absolute tolerance times the row length.
"""
import os

import numpy as np
import pytest

from tests import fused_op_cases as C

RTOL, ATOL = 1e-5, 1e-6


@pytest.fixture(scope="module")
def golden(golden_dir):
    return np.load(os.path.join(golden_dir, "fused_ops_golden.npz"))


def check_against_golden(golden, name, got):
    cols = golden["columns"]
    keys = [k.split("/")[1] for k in golden.files if k.startswith(name + "/") and not k.endswith("_rowsum")]
    assert sorted(keys) == sorted(got), (name, keys, sorted(got))
    for key in keys:
        a = np.asarray(got[key], dtype=np.float32)
        want = golden[f"{name}/{key}"]
        assert a[..., cols].shape == want.shape, (name, key)
        np.testing.assert_allclose(a[..., cols], want, rtol=RTOL, atol=ATOL, equal_nan=True, err_msg=f"{name}/{key}")
        mass = np.abs(a.astype(np.float64)).sum(-1)
        rs, want_rs = a.astype(np.float64).sum(-1), golden[f"{name}/{key}_rowsum"]
        # a sum of n entries that each agree to ATOL may differ by a fraction of n * ATOL (all-tie board: the
        # reference's tiled sums leave ~1e-7 per hand where prefix sums give exact zeros)
        slack = 1e-5 * mass + 1e-6 + 0.2 * ATOL * a.shape[-1]
        ok = (np.abs(rs - want_rs) <= slack) | (np.isnan(rs) & np.isnan(want_rs))
        assert ok.all(), (name, key, np.abs(rs - want_rs).max())


def test_fixture_lists_every_case(golden):
    assert tuple(golden["case_names"]) == C.NAMES


@pytest.mark.parametrize("name", C.NAMES)
def test_oracle_matches_reference_kernel_outputs(golden, name):
    check_against_golden(golden, name, C.oracle_ops(name, C.inputs(name)))


def test_fused_evaluator_switches_are_what_the_kernels_do(golden):
    """The three places where the oracle's ``fused_variant`` departs from the base evaluator,
    shown on the reference kernels' outputs themselves."""
    x = C.inputs("reach_and_deep_beliefs")
    tr, cols = x["tree"], golden["columns"]
    n = tr["bottom"]
    reach, beliefs = golden["reach_and_deep_beliefs/reach"], golden["reach_and_deep_beliefs/beliefs"]
    # the reach kernel writes child rows only: root rows keep their input (1 everywhere, blocked hands too)
    assert np.array_equal(reach[:n], x["reach"][:n][..., cols])
    assert (x["allowed"][:n] == 0).any()
    # the belief kernel skips the roots: they stay as given, not renormalised
    assert np.array_equal(beliefs[:n], x["beliefs"][:n][..., cols])
    # a child whose reach is all zero takes the prior row as it is handed in (row n+1 was zeroed)
    for player in (0, 1):
        assert np.array_equal(beliefs[n + 1, player], x["prob"][n + 1][cols])
    # average values: (avg * old + latest * new) * (1 / (old + new)), the reciprocal taken in fp32
    y = C.inputs("avg_values_zero_sum_off")
    inv = np.float32(1.0) / np.float32(y["old"] + y["new"])
    want = (y["avg"] * np.float32(y["old"]) + y["latest"] * np.float32(y["new"])) * inv
    np.testing.assert_allclose(golden["avg_values_zero_sum_off/avg"], want[..., cols], rtol=2e-7, atol=1e-7)
