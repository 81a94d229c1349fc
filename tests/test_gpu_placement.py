"""GPU: the placement aid (``p2hip_placement_probe``, ``p2hip_device_reserve`` / ``p2hip_device_release``)
and the evaluator's ``spread_state`` option, which deals the state tensors to two slabs and chooses the
second slab by the probe.  Placement is not arithmetic: a search with the option ends in exactly the state of
one without it, what was held goes back, and a block that does not fit is an error code, not a fault."""
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
    n = 48                                          # large enough for the probe: slabs of 100 MB and more
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


def test_placement_probe_through_the_c_abi():
    from poker2_amd import _lib
    lib = _lib.load()
    nbytes = 64 << 20
    a = torch.full((nbytes // 4,), 0.5, dtype=torch.float32, device="cuda")
    b = torch.full((nbytes // 4,), 0.25, dtype=torch.float32, device="cuda")
    ms = ctypes.c_float(-1.0)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.p2hip_placement_probe(a.data_ptr(), b.data_ptr(), nbytes, 2, ctypes.byref(ms), stream) == 0
    assert 0.0 < ms.value < 50.0
    # it streams rows of both buffers and overwrites part of them; everything stays finite and inside the buffers
    torch.cuda.synchronize()
    assert torch.isfinite(a).all() and torch.isfinite(b).all()
    assert not torch.equal(a, torch.full_like(a, 0.5)) or not torch.equal(b, torch.full_like(b, 0.25))
    # refused: no buffers, no result pointer, a repeat count out of range, buffers too small to say anything
    assert lib.p2hip_placement_probe(None, b.data_ptr(), nbytes, 2, ctypes.byref(ms), stream) != 0
    assert lib.p2hip_placement_probe(a.data_ptr(), b.data_ptr(), nbytes, 2, None, stream) != 0
    assert lib.p2hip_placement_probe(a.data_ptr(), b.data_ptr(), nbytes, 0, ctypes.byref(ms), stream) != 0
    assert lib.p2hip_placement_probe(a.data_ptr(), b.data_ptr(), 1 << 20, 2, ctypes.byref(ms), stream) != 0


def test_spread_state_changes_where_the_state_lies_and_nothing_else(monkeypatch):
    import poker2_amd.evaluator as E
    # the test's state is small: let the option apply to it, with steps that fit any card
    monkeypatch.setattr(E, "STATE_SPREAD_MIN_SLAB_BYTES", 32 << 20)
    monkeypatch.setattr(E, "STATE_SPREAD_STEP_BYTES", 63 << 20)
    monkeypatch.setattr(E, "STATE_SPREAD_TRIES", 3)
    torch.cuda.empty_cache()
    plain = _search(False, 0)
    assert plain.state_placement == {"placed": False}
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    cached_before = torch.cuda.memory_reserved()
    spread = _search(True, 0)
    p = spread.state_placement
    assert p["placed"] and 1 <= len(p["probe_ns_per_row_candidates"]) <= 3
    assert p["probe_ns_per_row_inside_first_slab"] > 0 and 0 <= p["chosen"] < len(p["probe_ns_per_row_candidates"])
    assert p["probe_ns_per_row_candidates"][p["chosen"]] == min(p["probe_ns_per_row_candidates"])
    for name in STATE:
        assert torch.equal(getattr(plain, name), getattr(spread, name)), name
    # the tensors of a side lie in one slab, neighbours in the dealing order in different slabs
    base = {spread.policy_probs.untyped_storage().data_ptr(), spread.policy_probs_avg.untyped_storage().data_ptr()}
    assert len(base) == 2
    assert spread.policy_probs_sample.untyped_storage().data_ptr() == spread.policy_probs.untyped_storage().data_ptr()
    assert spread.cumulative_regrets.untyped_storage().data_ptr() == spread.policy_probs_avg.untyped_storage().data_ptr()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    grown = torch.cuda.memory_reserved() - cached_before          # what the tensors' allocator took meanwhile
    assert (free_before - free_after) - grown < 16 << 20, "the held blocks were given back"


def test_a_second_subgame_on_the_same_evaluator_places_its_state_again(monkeypatch):
    import poker2_amd.evaluator as E
    monkeypatch.setattr(E, "STATE_SPREAD_MIN_SLAB_BYTES", 32 << 20)
    monkeypatch.setattr(E, "STATE_SPREAD_STEP_BYTES", 63 << 20)
    monkeypatch.setattr(E, "STATE_SPREAD_TRIES", 2)
    a = _search(True, 1)
    first = {name: getattr(a, name).clone() for name in STATE}
    b = _search(True, 1)
    assert a.state_placement["placed"] and b.state_placement["placed"]
    for name in STATE:
        assert torch.equal(first[name], getattr(b, name)), name


def _search_on(ev, seed: int, n: int, iterations: int = 9):
    from poker2_amd.tree import RootStates
    rng = np.random.default_rng(7400 + seed)
    boards = random_boards(rng, n)
    beliefs = random_ranges(rng, boards)
    roots = RootStates.at_round_start(3, rng.integers(40, 900, n), rng.integers(30, 2500, (n, 2)), boards,
                                      button=rng.integers(0, 2, n))
    ev.generator.manual_seed(5)                     # the sampling schedule is drawn per search
    ev.initialize_subgame(roots, np.arange(n), torch.from_numpy(beliefs))
    ev.evaluate_cfr()
    return {name: getattr(ev, name).clone() for name in STATE}


def _evaluator(n: int, **kw):
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    cfg = river_dcfr_config(n, iterations=9, depth=4, dcfr_delay=0)
    return HipSparseCFREvaluator(None, torch.device("cuda"), cfg, torch.Generator().manual_seed(5), max_raises=2, **kw)


@pytest.mark.parametrize("spread", [False, True])
def test_reuse_state_keeps_the_slabs_across_subgames_and_the_results(monkeypatch, spread):
    """``reuse_state``: successive subgames of one evaluator live in the same two slabs (replaced when a
    subgame needs more), and every one of them ends in the state a fresh evaluator reaches."""
    import poker2_amd.evaluator as E
    monkeypatch.setattr(E, "STATE_SPREAD_MIN_SLAB_BYTES", 32 << 20)
    monkeypatch.setattr(E, "STATE_SPREAD_STEP_BYTES", 63 << 20)
    monkeypatch.setattr(E, "STATE_SPREAD_TRIES", 2)
    sizes = [(0, 40), (1, 24), (2, 44), (3, 96), (4, 30)]        # second and third fit the first slabs; the fourth does not
    kept = _evaluator(40, reuse_state=True, spread_state=spread)
    slabs = []
    for seed, n in sizes:
        kept.cfg.num_envs = n
        got = _search_on(kept, seed, n)
        slabs.append(tuple(t.data_ptr() for t in kept._arena))
        want = _search_on(_evaluator(n), seed, n)
        for name in STATE:
            assert torch.equal(got[name], want[name]), (name, seed)
        assert kept.policy_probs.untyped_storage().data_ptr() == kept._arena[0].data_ptr()
        assert kept.policy_probs_avg.untyped_storage().data_ptr() == kept._arena[1].data_ptr()
    assert slabs[0] == slabs[1] == slabs[2], "subgames that fit keep the slabs"
    assert kept._arena[0].numel() >= 2 * 96 * 1326 * 4, "the large subgame got larger slabs"
    assert slabs[3] == slabs[4], "and the next small one stays in them"
    if spread:
        assert kept.state_placement["placed"] and kept.state_placement.get("reused")


def test_graph_replay_on_a_placed_state(monkeypatch):
    """A captured iteration (fused_cfr_triton.py:2359-2451) replays on state tensors that are views into
    the two slabs exactly as eager iterations run on separately allocated ones."""
    import poker2_amd.evaluator as E
    from poker2_amd.fused_cfr_hip import GraphedCFRIteration, _EvaluatorStateSnapshot
    from poker2_amd.tree import RootStates
    monkeypatch.setattr(E, "STATE_SPREAD_MIN_SLAB_BYTES", 32 << 20)
    monkeypatch.setattr(E, "STATE_SPREAD_STEP_BYTES", 63 << 20)
    monkeypatch.setattr(E, "STATE_SPREAD_TRIES", 2)
    n, iters = 48, 8
    rng = np.random.default_rng(7500)
    boards = random_boards(rng, n)
    beliefs = torch.from_numpy(random_ranges(rng, boards))
    roots = RootStates.at_round_start(3, rng.integers(40, 900, n), rng.integers(30, 2500, (n, 2)), boards,
                                      button=rng.integers(0, 2, n))

    def ready(**kw):
        ev = _evaluator(n, **kw)
        ev.initialize_subgame(roots, np.arange(n), beliefs)
        ev.prepare_search(t_sample=torch.full((ev.total_nodes,), 5, dtype=torch.long))
        return ev
    eager, graphed = ready(), ready(spread_state=True, reuse_state=True)
    assert graphed.state_placement["placed"] and not eager.state_placement["placed"]
    for t in range(3):
        eager.cfr_iteration(t)
        graphed.cfr_iteration(t)
    snap = _EvaluatorStateSnapshot.from_evaluator(graphed)
    runner = GraphedCFRIteration(graphed)
    runner.capture(t_capture=3, num_warmup=0)
    snap.restore_to(graphed)
    for t in range(3, iters):
        eager.cfr_iteration(t)
        runner.replay(t)
        torch.cuda.synchronize()
    for name in STATE:
        assert torch.equal(getattr(eager, name), getattr(graphed, name)), name


def test_placement_at_full_size_B1024_three_raise_tree():
    """BASELINE configuration 3's shape (1024 river roots, three-raise tree, 105 nodes per root) with the
    option's real constants - slabs of 5.8 and 4.8 GiB, steps of 31 GiB: the placed search ends in exactly
    the state of the search on tensors as allocated, and what was held is back on the card."""
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.tree import RootStates
    n = 1024
    rng = np.random.default_rng(77)
    boards = random_boards(rng, n)
    beliefs = torch.from_numpy(random_ranges(rng, boards))
    roots = RootStates.at_round_start(3, np.full(n, 200), np.tile([[800, 800]], (n, 1)), boards, button=np.arange(n) % 2)
    torch.cuda.empty_cache()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    states = []
    for spread in (False, True):
        ev = HipSparseCFREvaluator(None, torch.device("cuda"), river_dcfr_config(n, iterations=24, depth=16, dcfr_delay=0),
                                   torch.Generator().manual_seed(3), max_raises=3, spread_state=spread)
        ev.initialize_subgame(roots, np.arange(n), beliefs)
        assert ev.total_nodes == 105 * n
        ev.evaluate_cfr()
        p = ev.state_placement
        assert p["placed"] == spread
        if spread:
            assert 1 <= len(p["probe_ns_per_row_candidates"]) <= 6 and 5.0 < p["probe_ns_per_row_inside_first_slab"] < 200.0
            assert min(p["probe_ns_per_row_candidates"]) <= 1.05 * p["probe_ns_per_row_inside_first_slab"]
            print("placement at B=1024:", {k: (round(v, 2) if isinstance(v, float) else v) for k, v in p.items()})
        states.append({name: getattr(ev, name).clone() for name in STATE})
        del ev
    for name in STATE:
        assert torch.equal(states[0][name], states[1][name]), name
    del states
    torch.cuda.empty_cache()
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_before - free_after < 1 << 30, "slabs, candidates and held blocks are back on the card"
