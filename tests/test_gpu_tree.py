"""GPU: the device tree builder against the host builder (itself pinned by fixtures written from
the reference's HUNLTensorEnv, tests/test_tree.py): every array identical, bit for bit."""
import numpy as np
import pytest

from tests.helpers import random_boards

pytestmark = pytest.mark.gpu

FIELDS = ("parent_index", "action_from_parent", "child_count", "child_offsets", "prev_actor", "root_index",
          "legal_mask", "leaf_mask", "new_street_mask", "fold_mask", "showdown_mask", "reward", "board")


def same_tree(a, b):
    assert a.depth_offsets == b.depth_offsets and a.total == b.total and a.num_actions == b.num_actions
    for name in FIELDS:
        x, y = getattr(a, name), getattr(b, name)
        assert x.dtype == y.dtype and x.shape == y.shape, name
        assert np.array_equal(x, y), name
    assert set(a.state) == set(b.state)
    for name in a.state:
        x, y = a.state[name], b.state[name]
        assert x.dtype == y.dtype and np.array_equal(x, y), name


def random_roots(rng, n, street):
    from poker2_amd.tree import RootStates
    k = {1: 3, 2: 4, 3: 5, 0: 0}[street]
    boards = np.full((n, 5), -1, dtype=np.int64)
    if k:
        boards[:, :k] = random_boards(rng, n, k)
    pot = rng.integers(20, 600, n)
    stacks = rng.integers(0, 3, (n, 2)) * rng.integers(50, 1500, (n, 2)) + rng.integers(1, 900, (n, 2))
    return RootStates.at_round_start(street, pot, stacks, boards, button=rng.integers(0, 2, n), bb=rng.choice([10, 100]))


@pytest.mark.parametrize("street,bins,depth,max_raises", [
    (3, [0.5, 1.0], 2, None), (3, [0.5, 1.0], 16, 3), (2, [0.33, 0.75, 1.5], 4, None), (1, [1.0], 6, 2),
    (3, [], 5, None), (2, [0.25, 0.5, 1.0, 2.0, 4.0], 3, None)])
def test_device_builder_equals_host_builder(street, bins, depth, max_raises):
    from poker2_amd.tree import build_sparse_tree, build_sparse_tree_device
    rng = np.random.default_rng(100 * street + depth)
    roots = random_roots(rng, 300, street)
    host = build_sparse_tree(roots, bins, depth, max_raises=max_raises)
    dev = build_sparse_tree_device(roots, bins, depth, max_raises=max_raises)
    same_tree(host, dev)
    for name, t in dev.device_arrays.items():
        ref = getattr(host, name) if name in FIELDS + ("showdown_potential",) else host.state[name]
        got = t.cpu().numpy()
        assert got.dtype == np.asarray(ref).dtype and np.array_equal(got, ref), name


def test_device_builder_from_mid_round_roots():
    """Roots in the middle of a betting round (chips committed, a raise made, one player all-in):
    the non-terminal nodes of another tree."""
    from poker2_amd.tree import RootStates, build_sparse_tree, build_sparse_tree_device
    rng = np.random.default_rng(7)
    first = build_sparse_tree(random_roots(rng, 60, 2), [0.5, 1.0], 3)
    rows = np.nonzero(~first.state["done"])[0]
    fields = {}
    for name in RootStates.__dataclass_fields__:
        if name == "board":
            fields[name] = first.board[first.root_index[rows]]
        elif name == "bb":
            fields[name] = 100
        elif name in ("last_board", "runout"):
            fields[name] = None
        else:
            fields[name] = np.asarray(first.state[name])[rows]
    roots = RootStates(**fields)
    assert roots.is_allin.any() and (roots.committed.sum(1) > 0).any()
    same_tree(build_sparse_tree(roots, [0.5, 1.0], 4, max_raises=2),
              build_sparse_tree_device(roots, [0.5, 1.0], 4, max_raises=2))


def test_device_builder_from_preflop_roots():
    """Roots as the environment's reset leaves them: blinds committed, the button to act."""
    from poker2_amd.tree import RootStates, build_sparse_tree, build_sparse_tree_device
    rng = np.random.default_rng(11)
    n = 200
    roots = RootStates.preflop(n, starting_stacks=rng.integers(150, 20000, (n, 2)), button=rng.integers(0, 2, n))
    same_tree(build_sparse_tree(roots, [0.5, 1.0], 5, max_raises=3),
              build_sparse_tree_device(roots, [0.5, 1.0], 5, max_raises=3))


def test_device_builder_on_the_reference_env_fixture(golden_dir):
    """Every case of tests/golden/tree_golden.npz (written by the reference's HUNLTensorEnv: river,
    turn, flop and reset-state roots, three bin sets, depths 2-12, the 50 / 100 and the 5 / 10
    blinds) straight through the device builder."""
    from poker2_amd.tree import build_sparse_tree_device
    from tests.test_tree import STATE_KEYS, cases, roots_of
    seen = 0
    for name, case in cases(golden_dir):
        roots, _, _ = roots_of(case)
        t = build_sparse_tree_device(roots, [float(x) for x in case["bins"]], int(case["depth"]))
        assert t.depth_offsets == list(case["depth_offsets"]), name
        assert np.array_equal(t.parent_index, case["parent_index"]), name
        assert np.array_equal(t.action_from_parent, case["action_from_parent"]), name
        assert np.array_equal(t.legal_mask, case["legal_mask"]), name
        for k in STATE_KEYS:
            assert np.array_equal(t.state[k], case[k].astype(t.state[k].dtype)), (name, k)
        assert np.array_equal(t.reward[t.fold_mask], case["reward"][t.fold_mask]), name
        seen += 1
    assert seen >= 9
