"""GPU: the placement aid (``p2hip_device_reserve`` / ``p2hip_device_release``) and the evaluator's
``spread_state`` option, which allocates each state tensor while such a block is held.  Placement is
not arithmetic: a search with the option ends in exactly the state of one without it, the blocks are
given back, and a block that does not fit is an error code, not a fault."""
import ctypes

import numpy as np
import pytest
import torch

from tests.helpers import random_boards, random_ranges

pytestmark = pytest.mark.gpu

STATE = ("policy_probs", "policy_probs_avg", "policy_probs_sample", "cumulative_regrets", "regret_weight_sums",
         "self_reach", "self_reach_avg", "beliefs", "beliefs_avg", "latest_values", "values_avg")


def test_reserve_and_release_through_the_c_abi():
    from poker2_amd import _lib
    lib = _lib.load()
    torch.zeros(1, device="cuda")
    torch.cuda.synchronize()
    free_before, total = torch.cuda.mem_get_info()
    block = ctypes.c_void_p()
    assert lib.p2hip_device_reserve(64 << 20, ctypes.byref(block)) == 0 and block.value
    free_held, _ = torch.cuda.mem_get_info()
    assert free_before - free_held >= 64 << 20
    assert lib.p2hip_device_release(block) == 0
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after >= free_before - (2 << 20)
    assert lib.p2hip_device_release(None) == 0                       # nothing to release
    # refused requests: an error code and no block
    for bad in (0, -5):
        block = ctypes.c_void_p(1)
        assert lib.p2hip_device_reserve(bad, ctypes.byref(block)) != 0 and not block.value
    assert lib.p2hip_device_reserve(1 << 20, None) != 0
    block = ctypes.c_void_p(1)
    assert lib.p2hip_device_reserve(4 * total, ctypes.byref(block)) != 0 and not block.value   # does not fit
    # and nothing is left pending: the next HIP work runs
    x = torch.arange(1000, device="cuda").sum()
    assert int(x) == 499500


def _search(spread: bool, seed: int):
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.tree import RootStates
    rng = np.random.default_rng(7300 + seed)
    n = 6
    boards = random_boards(rng, n)
    beliefs = random_ranges(rng, boards)
    roots = RootStates.at_round_start(3, rng.integers(40, 900, n), rng.integers(30, 2500, (n, 2)), boards,
                                      button=rng.integers(0, 2, n))
    cfg = river_dcfr_config(n, iterations=9, depth=4, dcfr_delay=0)
    ev = HipSparseCFREvaluator(None, torch.device("cuda"), cfg, torch.Generator().manual_seed(5), max_raises=2,
                               spread_state=spread)
    ev.initialize_subgame(roots, np.arange(n), torch.from_numpy(beliefs))
    ev.evaluate_cfr()
    return ev


def test_spread_state_changes_where_the_state_lies_and_nothing_else(monkeypatch):
    import poker2_amd.evaluator as E
    # the test's tensors are small: let the option apply to them, with a block that fits any card
    monkeypatch.setattr(E, "STATE_SPREAD_MIN_TENSOR_BYTES", 0)
    monkeypatch.setattr(E, "STATE_SPREAD_GAP_BYTES", 48 << 20)
    torch.cuda.empty_cache()
    plain = _search(False, 0)
    assert plain.state_spread_count == 0
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    cached_before = torch.cuda.memory_reserved()
    spread = _search(True, 0)
    # cached blocks of the allocator may serve some of the tensors; the others went behind a block
    assert 0 <= spread.state_spread_count <= 13
    for name in STATE:
        assert torch.equal(getattr(plain, name), getattr(spread, name)), name
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    grown = torch.cuda.memory_reserved() - cached_before          # what the tensors' allocator took meanwhile
    assert (free_before - free_after) - grown < 16 << 20, "the held blocks were given back"


def test_spread_state_places_tensors_when_the_allocator_has_nothing_cached(monkeypatch):
    import poker2_amd.evaluator as E
    monkeypatch.setattr(E, "STATE_SPREAD_MIN_TENSOR_BYTES", 0)
    monkeypatch.setattr(E, "STATE_SPREAD_GAP_BYTES", 48 << 20)
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    ev = HipSparseCFREvaluator(None, torch.device("cuda"), river_dcfr_config(1, iterations=2, depth=2), spread_state=True)
    torch.cuda.empty_cache()
    # large enough that no cached small-pool block serves it
    t = ev._new_state(3000, 2, 1326)
    assert ev.state_spread_count == 1 and float(t.abs().sum()) == 0.0
    off = HipSparseCFREvaluator(None, torch.device("cuda"), river_dcfr_config(1, iterations=2, depth=2))
    off._new_state(3000, 2, 1326)
    assert off.state_spread_count == 0
