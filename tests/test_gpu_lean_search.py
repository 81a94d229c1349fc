"""GPU: a search whose iterations run lean (rows nobody reads before the next iteration are not
stored; reach_avg alternates between two buffers) ends in exactly the state of a search whose
iterations all run as ``cfr_iteration`` runs them: ``torch.equal`` on all eleven tensors, over random
trees, every CFR variant, leaf models, work items on and off, odd and even iteration counts.  Which
rows may be skipped is shown on the CPU oracle (tests/test_oracle_lean_rows.py); here the skipped rows
are additionally overwritten with NaN between iterations, so a single read of one would show."""
import ctypes

import numpy as np
import pytest
import torch

from tests.helpers import random_boards, random_ranges

pytestmark = pytest.mark.gpu

STATE = ("policy_probs", "policy_probs_avg", "policy_probs_sample", "cumulative_regrets", "regret_weight_sums",
         "self_reach", "self_reach_avg", "beliefs", "beliefs_avg", "latest_values", "values_avg")
VARIANTS = [  # cfr_type, delay, cfr_plus, cfr_avg, model (None | "zero_sum" | "plain")
    ("discounted", 0, False, False, None),
    ("discounted", 3, False, False, "plain"),
    ("discounted_plus", 2, True, False, None),
    ("standard", 0, False, False, "zero_sum"),
    ("linear", 0, False, False, None),
    ("discounted", 0, False, True, "plain"),
    ("linear", 0, False, True, "zero_sum"),
    ("linear", 0, True, False, "plain"),
]


def build(seed, variant, split, lean, iters):
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.fused_cfr_hip import CFRType
    from poker2_amd.tree import RootStates
    cfr_type, delay, cfr_plus, cfr_avg, model_kind = variant
    rng = np.random.default_rng(9100 + seed)
    n = int(rng.integers(1, 6))
    bins = sorted(rng.choice([0.25, 0.5, 0.75, 1.0, 2.0], size=int(rng.integers(1, 5)), replace=False).tolist())
    depth = int(rng.integers(2, 6))
    max_raises = [None, 2, 3][int(rng.integers(0, 3))]
    street = 2 if seed % 2 else 3
    boards = random_boards(rng, n)
    if street == 2:
        boards[:, 4] = -1
    beliefs = random_ranges(rng, boards)
    roots = RootStates.at_round_start(street, rng.integers(40, 900, n), rng.integers(30, 2500, (n, 2)), boards,
                                      button=rng.integers(0, 2, n), bb=int(rng.choice([10, 100])))
    model = None
    if model_kind is not None:
        class LeafModel:                       # a deterministic stand-in for the value network
            enforce_zero_sum = model_kind == "zero_sum"

            def leaf_values(self, bel, rows, ev):
                return 0.3 * torch.flip(bel, dims=[1]) * 50.0 - 0.01
        model = LeafModel()
    cfg = river_dcfr_config(n, iterations=iters, depth=depth, dcfr_delay=delay)
    cfg.search.cfr_type = CFRType[cfr_type]
    cfg.search.cfr_plus, cfg.search.cfr_avg = cfr_plus, cfr_avg
    cfg.env.bet_bins = bins
    ev = HipSparseCFREvaluator(model, torch.device("cuda"), cfg, max_raises=max_raises, split_small_batches=split,
                               lean_search=lean)
    ev.initialize_subgame(roots, np.arange(n), torch.from_numpy(beliefs))
    t_sample = torch.from_numpy(rng.integers(0, iters, n))[torch.from_numpy(ev.tree.root_index)]
    ev.prepare_search(t_sample=t_sample)
    return ev


def dead_rows(ev) -> dict:
    """The rule of tests/test_oracle_lean_rows.py on the product's tree."""
    tree = ev.tree
    below_root = np.arange(tree.total) >= tree.n_roots
    parent = tree.child_count > 0
    leaf_eval = tree.showdown_mask.copy()
    if ev.model is not None:
        leaf_eval |= tree.leaf_mask & ~np.asarray(tree.state["done"])
    keep_b = parent | (leaf_eval & (not ev.cfr_avg))
    if ev.enforce_zero_sum:
        keep_ba = np.ones(tree.total, bool)
    elif ev.cfr_avg:
        keep_ba = parent | leaf_eval
    else:
        keep_ba = np.zeros(tree.total, bool)
    masks = {"self_reach": below_root & ~parent, "self_reach_avg": below_root & ~parent,
             "beliefs": below_root & ~keep_b, "beliefs_avg": below_root & ~keep_ba}
    return {k: torch.from_numpy(m).to(ev.device) for k, m in masks.items()}


@pytest.mark.parametrize("split", [False, True])
@pytest.mark.parametrize("seed", range(8))
def test_lean_search_ends_in_the_state_of_a_plain_search(seed, split):
    variant = VARIANTS[seed % len(VARIANTS)]
    iters = 5 + seed % 2                                   # odd and even: the alternation ends where it started
    plain = build(seed, variant, split, lean=False, iters=iters)
    lean = build(seed, variant, split, lean=True, iters=iters)
    assert split or lean._items is None
    home = lean.self_reach_avg
    plain.run_search_iterations()
    lean.run_search_iterations()
    assert lean.self_reach_avg is home
    for name in STATE:
        assert torch.equal(getattr(plain, name), getattr(lean, name)), f"seed {seed} {variant} split {split}: {name}"
    # the searches' outputs built on top of the state agree as well
    assert torch.equal(plain._compute_exploitability().local_exploitability,
                       lean._compute_exploitability().local_exploitability)


@pytest.mark.parametrize("seed", range(8))
def test_rows_a_lean_iteration_skips_are_never_read(seed):
    variant = VARIANTS[(seed + 3) % len(VARIANTS)]
    iters = 6 - seed % 2
    plain = build(seed, variant, bool(seed % 2), lean=False, iters=iters)
    lean = build(seed, variant, bool(seed % 2), lean=True, iters=iters)
    dead = dead_rows(lean)
    for t in range(iters):
        plain.cfr_iteration(t)
        last = t + 1 == iters
        lean.cfr_iteration(t, lean=not last, alternate_reach_avg=not (iters % 2 == 1 and t == 0))
        if not last:
            for name, mask in dead.items():
                getattr(lean, name)[mask] = float("nan")
            # what the other reach_avg buffer still holds is two iterations old: nothing may read it either
            if lean._reach_avg_alt is not None:
                lean._reach_avg_alt[lean.root_nodes:] = float("nan")
                # ... except that it is the buffer the next alternating iteration writes before it reads
    for name in STATE:
        got = getattr(lean, name)
        assert bool(torch.isfinite(got).all()), name
        assert torch.equal(getattr(plain, name), got), f"seed {seed} {variant}: {name}"


def test_entry_point_refuses_inconsistent_modes():
    from poker2_amd import _lib
    ev = build(0, VARIANTS[0], False, lean=True, iters=4)
    args = ev._iter_bundle(False).main
    lib = _lib.load()
    stream = _lib.stream_ptr()
    assert lib.p2hip_cfr_iteration(ctypes.byref(args), ev.root_nodes, ev._max_children, 16, stream) != 0   # lean, but no sweep
    assert lib.p2hip_cfr_iteration(ctypes.byref(args), ev.root_nodes, ev._max_children, 32 | 3, stream) != 0
    bad = ev._build_iter_args(reach_avg=ev.self_reach_avg, reach_avg_prev=ev.self_reach_avg)
    assert lib.p2hip_cfr_iteration(ctypes.byref(bad), ev.root_nodes, ev._max_children, 3, stream) != 0     # in place AND previous
    torch.cuda.synchronize()
