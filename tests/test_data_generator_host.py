"""CPU: host-side pieces of data generation that need no GPU — dealing new hands like the
reference env's reset (src/p2/env/hunl_tensor_env.py:219-346), the previous-board rule, the batch
container (src/p2/rl/rebel_batch.py:16-70, 127-167)."""
import numpy as np
import pytest
import torch

from poker2_amd.chance_node_helper import MLPFeatures
from poker2_amd.rebel_batch import RebelBatch
from poker2_amd.rebel_data_generator import EnvProto
from poker2_amd.tree import RootStates

H = 1326


def test_reset_deals_the_hands_the_reference_env_deals(golden_dir):
    g = np.load(str(golden_dir) + "/training_data_golden.npz")
    gen = torch.Generator(device="cpu")
    gen.manual_seed(int(g["reset/seed"]))
    proto = EnvProto(mean_stack=1000, sb=50, bb=100, randomize_stacks=True, rng=gen)
    roots = proto.reset(16)
    assert np.array_equal(proto.last_deck, g["reset/deck"])
    assert np.array_equal(roots.runout, g["reset/deck"][:, 4:9])
    for name in ("street", "to_act", "button", "pot", "stacks", "committed", "min_raise", "actions_this_round",
                 "is_allin", "starting_stacks", "scale", "done"):
        assert np.array_equal(getattr(roots, name), g[f"reset/{name}"]), name
    assert np.array_equal(roots.board, g["reset/board_indices"])
    assert np.array_equal(roots.previous_board(), g["reset/last_board_indices"])


def test_previous_board_rule_on_the_reference_roots(golden_dir):
    g = np.load(str(golden_dir) + "/training_data_golden.npz")
    for case in ("streets_mixed", "preflop"):
        r = {k.split("/")[-1]: g[k] for k in g.files if k.startswith(case + "/root/")}
        n = len(r["street"])
        roots = RootStates(street=r["street"], to_act=r["to_act"], button=r["button"], pot=r["pot"],
                           stacks=r["stacks"], committed=r["committed"], min_raise=r["min_raise"],
                           actions_this_round=r["actions_this_round"], is_allin=r["is_allin"],
                           starting_stacks=r["starting_stacks"], scale=r["scale"], board=r["board_indices"])
        assert np.array_equal(roots.previous_board(), r["last_board_indices"]), case
        assert roots.n == n


def test_runout_must_continue_the_board():
    board = np.array([[1, 2, 3, -1, -1]])
    kw = dict(street=np.array([1]), to_act=np.array([0]), button=np.array([1]), pot=np.array([200]),
              stacks=np.array([[900, 900]]), committed=np.zeros((1, 2), np.int64), min_raise=np.array([100]),
              actions_this_round=np.array([0]), is_allin=np.zeros((1, 2), bool),
              starting_stacks=np.array([[1000, 1000]]), scale=np.array([1000.0], np.float32), board=board)
    RootStates(**kw, runout=np.array([[1, 2, 3, 9, 10]]))
    with pytest.raises(AssertionError):
        RootStates(**kw, runout=np.array([[1, 2, 4, 9, 10]]))


def features(n, seed):
    g = torch.Generator().manual_seed(seed)
    return MLPFeatures(context=torch.rand(n, 4, generator=g), street=torch.zeros(n), to_act=torch.zeros(n, dtype=torch.long),
                       board=torch.full((n, 5), -1), beliefs=torch.rand(n, 2 * H, generator=g))


def test_batch_indexing_and_concatenation():
    a = RebelBatch(features=features(3, 0), legal_masks=torch.ones(3, 5, dtype=torch.bool),
                   value_targets=torch.rand(3, 2, H), statistics={"pot": torch.tensor([1, 2, 3])})
    b = RebelBatch(features=features(0, 1), legal_masks=torch.ones(0, 5, dtype=torch.bool),
                   value_targets=torch.rand(0, 2, H), statistics={"pot": torch.zeros(0, dtype=torch.long)})
    c = RebelBatch.cat([a, b, a[torch.tensor([True, False, True])]])
    assert len(c) == 5 and c.statistics["pot"].tolist() == [1, 2, 3, 1, 3]
    assert torch.equal(c.features.beliefs[3], a.features.beliefs[0]) and c.policy_targets is None
    p = RebelBatch(features=features(2, 2), legal_masks=torch.ones(2, 5, dtype=torch.bool), policy_targets=torch.rand(2, H, 5))
    with pytest.raises(ValueError):
        RebelBatch.cat([a, p])                      # value targets must be all present or all absent
    with pytest.raises(ValueError):
        RebelBatch.cat([])
    with pytest.raises(AssertionError):
        RebelBatch(features=features(2, 3), legal_masks=torch.ones(2, 5, dtype=torch.bool))   # no targets at all
    with pytest.raises(AssertionError):
        RebelBatch(features=features(2, 3), legal_masks=torch.ones(3, 5, dtype=torch.bool), value_targets=torch.rand(2, 2, H))


# ---- the generator loop on a stand-in evaluator (the cases of the reference's
# tests/test_rebel_data_generator.py:204-320) -----------------------------------------------------
class DummyEvaluator:
    """Records how the loop drives it; returns fixed batches."""

    def __init__(self, n, returns):
        self.root_nodes, self.num_players, self.device = n, 2, torch.device("cpu")
        self.returns = list(returns)          # what evaluate_cfr hands back, call by call
        self.initialize_args, self.evaluate_calls = [], 0

    def initialize_subgame(self, env, indices, beliefs):
        assert env.n == self.root_nodes and beliefs.shape == (self.root_nodes, 2, H)
        self.initialize_args.append((env, np.asarray(indices).copy(), beliefs.clone()))

    def evaluate_cfr(self):
        self.evaluate_calls += 1
        return self.returns.pop(0) if self.returns else None

    def training_data(self):
        n = self.root_nodes
        value = RebelBatch(features=features(n, 1), legal_masks=torch.ones(n, 5, dtype=torch.bool),
                           value_targets=torch.full((n, 2, H), 0.25))
        pre = value[torch.zeros(n, dtype=torch.bool)]
        policy = RebelBatch(features=features(n, 2), legal_masks=torch.ones(n, 5, dtype=torch.bool),
                            policy_targets=torch.full((n, H, 5), 0.2))
        return value, pre, policy


class ListBuffer:
    def __init__(self):
        self.batches = []

    def add_batch(self, b):
        self.batches.append(b)


def make_generator(n, returns, seed=3):
    from poker2_amd.rebel_data_generator import RebelDataGenerator
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    ev = DummyEvaluator(n, returns)
    buf = ListBuffer()
    return RebelDataGenerator(EnvProto(1000, rng=gen), ev, buf, buf), ev, buf


def test_generator_collects_and_orders_batches():
    dg, ev, buf = make_generator(2, [])
    value, policy = dg.generate_data(2)
    # one search was enough; policy batch goes to its buffer first, then the two value batches
    assert ev.evaluate_calls == 1 and len(buf.batches) == 3
    assert buf.batches[0].policy_targets is not None and buf.batches[1].value_targets is not None
    assert len(buf.batches[2]) == 0
    assert np.array_equal(ev.initialize_args[0][1], np.arange(2))
    assert torch.allclose(ev.initialize_args[0][2], torch.full((2, 2, H), 1.0 / H))     # fresh hands: uniform ranges
    assert (ev.initialize_args[0][0].street == 0).all()
    assert len(value) == 2 and len(policy) == 2 and dg.last_extra == 0
    assert dg.current_pbs is None                       # the search had no states to continue from


def test_generator_restarts_from_fresh_hands_and_counts_surplus():
    dg, ev, buf = make_generator(4, [None, None])
    dg.generate_data(6)                                  # 4 + 4 samples for 6 asked: 2 carried over
    assert ev.evaluate_calls == 2 and dg.last_extra == 2
    assert all((args[0].street == 0).all() for args in ev.initialize_args)
    dg.generate_data(2)                                  # already covered by the surplus
    assert ev.evaluate_calls == 2 and dg.last_extra == 0


def test_generator_continues_sampled_states_and_refills():
    from poker2_amd.rebel_data_generator import PublicBeliefState
    n = 4
    # two states come back from the first search: flop states with their runout and skewed ranges
    runout = np.array([[1, 2, 3, 4, 5], [10, 20, 30, 40, 50]])
    board = runout.copy()
    board[:, 3:] = -1
    cont = RootStates.at_round_start(1, [300, 500], [[850, 850], [750, 750]], board, button=[1, 0])
    cont.runout = runout
    bel = torch.rand(2, 2, H)
    dg, ev, buf = make_generator(n, [PublicBeliefState(env=cont, beliefs=bel), None])
    dg.generate_data(2 * n)
    assert ev.evaluate_calls == 2
    env2, _, bel2 = ev.initialize_args[1]
    assert env2.n == n
    assert env2.street.tolist()[:2] == [1, 1] and (env2.street[2:] == 0).all()           # continued, then fresh hands
    assert np.array_equal(env2.board[:2], board) and (env2.board[2:] == -1).all()
    assert np.array_equal(env2.runout[:2], runout)
    assert np.array_equal(env2.previous_board()[:2], np.full((2, 5), -1))                 # flop just dealt
    assert env2.pot.tolist()[:2] == [300, 500] and (env2.pot[2:] == 150).all()
    assert torch.equal(bel2[:2], bel) and torch.allclose(bel2[2:], torch.full((2, 2, H), 1.0 / H))
