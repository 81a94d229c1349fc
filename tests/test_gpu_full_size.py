"""GPU: the two largest configurations at their real batch sizes, checked through properties that
do not depend on the size — probabilities sum to one, targets stay in range, and a root's result
does not depend on which other roots share its batch (the search shares nothing between roots).

  turn subgames with chance leaves: 512 four-card boards, every street-end leaf expanded over
      the 48 river cards and evaluated by the 3 x 1536 fp32 network;
  one data-generation step: 16 384 mixed flop / turn / river roots searched to the end of the
      street with the bf16 network at the leaves, then ``training_data``.
Few iterations: the size is what these tests are about."""
import numpy as np
import pytest
import torch

from tests.helpers import H, random_boards, random_ranges

pytestmark = pytest.mark.gpu
DEV = "cuda"


def sibling_sums(ev, policy, parents):
    """Sum of ``policy`` over the children of each of ``parents`` -> [len(parents), H]."""
    out = torch.empty(len(parents), H, device=DEV)
    first, count = ev.child_offsets[parents].tolist(), ev.child_count[parents].tolist()
    for i, (f, c) in enumerate(zip(first, count)):
        out[i] = policy[f:f + c].sum(0)
    return out


def check_distributions(ev, rng, n_sample=256):
    top = ev.depth_offsets[-2]
    parents = torch.nonzero(ev.child_count[:top] > 0).flatten()
    pick = parents[torch.from_numpy(rng.choice(len(parents), min(n_sample, len(parents)), replace=False)).to(DEV)]
    for pol in (ev.policy_probs, ev.policy_probs_avg):
        s = sibling_sums(ev, pol, pick)
        torch.testing.assert_close(s, torch.ones_like(s), rtol=0, atol=2e-5)
    rows = torch.from_numpy(rng.choice(ev.total_nodes, n_sample, replace=False)).to(DEV)
    for b in (ev.beliefs, ev.beliefs_avg):
        s = b[rows].sum(-1)
        torch.testing.assert_close(s, torch.ones_like(s), rtol=0, atol=2e-5)
    assert torch.isfinite(ev.values_avg).all() and torch.isfinite(ev.latest_values).all()


def same_but_few(big, ref, name, rtol=1e-3, atol=2e-4):
    """The network's GEMMs run at another batch size (another hipBLASLt tiling), so leaf values
    agree to ~1e-6 only, and regret matching sits on top of them: all entries within tolerance
    except at most max(2, 1e-4 of them), none of those off by more than 1e-2.  Values are compared
    where they are in range: on hands that face (almost) no compatible opponent hand the showdown
    quotient is rounding noise on both sides."""
    a, b = big.float(), ref.float()
    if name == "values_avg":
        keep = b.abs() <= 1.0
        a, b = a[keep], b[keep]
    diff = (a - b).abs()
    over = diff > atol + rtol * b.abs()
    n_over = int(over.sum())
    assert n_over <= max(2, 1e-4 * diff.numel()) and (n_over == 0 or float(diff[over].max()) < 1e-2), \
        f"{name}: {n_over} of {diff.numel()} over tolerance, max abs diff {float(diff.max()):.3e}"


class RowWiseNetwork:
    """A stand-in for the value network whose answer for a sample depends on that sample alone and has no
    sum in it (the opponent's range, scaled by the board's ranks): no GEMM tiling, so a root's search
    must give the same bits whatever batch it is part of."""

    def eval(self):
        pass

    def __call__(self, f, include_policy=False):
        from types import SimpleNamespace
        b = f.beliefs.view(-1, 2, H).float()
        ranks = torch.where(f.board >= 0, (f.board % 13).float(), torch.zeros_like(f.board, dtype=torch.float32))
        return SimpleNamespace(hand_values=torch.flip(b, dims=[1]) * (40.0 + ranks.sum(dim=1))[:, None, None] - 0.01)


STATE_TENSORS = ("policy_probs", "policy_probs_avg", "policy_probs_sample", "cumulative_regrets", "regret_weight_sums",
                 "self_reach", "self_reach_avg", "beliefs", "beliefs_avg", "latest_values", "values_avg")


def rows_of_first_roots(ev, k):
    """Node rows that belong to roots 0..k-1, in row order (= the row order of a tree built from
    those roots alone: rows are level-major, parent-major)."""
    return np.nonzero(ev.tree.root_index < k)[0]


def test_turn_subgames_with_chance_leaves_B512():
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.leaf_models import ChanceLeafModel, RangeBoardMLP
    from poker2_amd.tree import RootStates
    rng = np.random.default_rng(404)
    b, small, iters = 512, 6, 3
    boards = random_boards(rng, b, 5)
    boards[:, 4] = -1
    beliefs = random_ranges(rng, boards)
    dev = torch.device(DEV)
    net = RangeBoardMLP().to(dev)                       # 2 x 1326 + 52 -> 3 x 1536 ReLU -> 2 x 1326, fp32
    with torch.no_grad():
        for lin in net.linears:
            lin.weight.mul_(2.0)

    def run(n, iters=iters, network=net):
        roots = RootStates.at_round_start(2, np.full(n, 200), np.tile([[800, 800]], (n, 1)), boards[:n],
                                          button=np.arange(n) % 2)
        # the configuration's own bet tree: bins {0.5, 1} pot + all-in, at most three raises
        ev = HipSparseCFREvaluator(ChanceLeafModel(network, dev), dev, river_dcfr_config(n, iterations=iters, depth=16,
                                                                                         dcfr_delay=0), max_raises=3)
        ev.initialize_subgame(roots, np.arange(n), torch.from_numpy(beliefs[:n]))
        ev.prepare_search(t_sample=torch.full((ev.total_nodes,), -1, dtype=torch.long))
        ev.run_search_iterations()
        return ev
    # the configuration's own length: 100 iterations at the full batch, checked by what every state must satisfy
    ev = run(b, 100)
    assert ev.total_nodes == 105 * b and ev.model_indices.numel() == 35 * b      # 35 street-end leaves per root
    assert float(ev.latest_values[ev.model_indices].abs().max()) > 1e-3          # the network matters
    check_distributions(ev, rng)
    stats = ev._compute_exploitability()
    assert torch.isfinite(stats.local_exploitability).all() and float(stats.local_exploitability.min()) > -1e-4
    del ev, stats
    # batch independence over a few iterations (longer runs of two float32 programs drift apart on their own)
    ev = run(b)
    check_distributions(ev, rng)
    ref = run(small)
    rows = rows_of_first_roots(ev, small)
    assert len(rows) == ref.total_nodes
    rows = torch.from_numpy(rows).to(DEV)
    for name in ("policy_probs_avg", "beliefs_avg", "values_avg"):
        same_but_few(getattr(ev, name)[rows], getattr(ref, name), name)
    del ev, ref
    # the same with a network that has no GEMM in it: every tensor of the first roots bit for bit, so the tolerance
    # above is the network's and not the library's (expansion, mean and iteration do not depend on the batch)
    ev = run(b, 6, RowWiseNetwork())
    ref = run(small, 6, RowWiseNetwork())
    assert float(ev.latest_values[ev.model_indices].abs().max()) > 1e-3
    for name in STATE_TENSORS:
        assert torch.equal(getattr(ev, name)[rows], getattr(ref, name)), name


def test_data_generation_step_B16384():
    from poker2_amd.bench_datagen import make_roots
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.leaf_models import NetworkLeafModel, RangeBoardMLP
    rng = np.random.default_rng(405)
    b, small, iters = 16384, 24, 4
    roots, bel = make_roots(b, 5)
    dev = torch.device(DEV)
    net = RangeBoardMLP().to(dev)
    with torch.no_grad():
        for lin in net.linears:
            lin.weight.mul_(2.0)

    def run(n, autocast, iters=iters, network=net):
        gen = torch.Generator(device=dev)
        gen.manual_seed(1)
        model = NetworkLeafModel(network, dev, autocast_dtype=autocast)
        ev = HipSparseCFREvaluator(model, dev, river_dcfr_config(n, iterations=iters, depth=64), generator=gen,
                                   max_raises=3)
        ev.initialize_subgame(roots.select(np.arange(n)), np.arange(n), bel[:n])
        nxt = ev.evaluate_cfr()
        return ev, nxt
    ev, nxt = run(b, torch.bfloat16, 64)                                          # the configuration's own 64 iterations
    assert ev.total_nodes > 20 * b and ev.model_indices.numel() > b and ev.showdown_indices.numel() > b
    check_distributions(ev, rng)
    assert nxt.roots.n == b                                                       # one sampled leaf per root
    street = np.asarray(nxt.roots.street)
    dealt = (np.asarray(nxt.roots.board) >= 0).sum(1)
    assert ((dealt == np.array([0, 3, 4, 5, 5])[street]) | np.asarray(nxt.roots.done)).all()   # cards match the street
    ev.chance_helper.autocast_dtype = torch.bfloat16
    value, pre_value, policy = ev.training_data()
    assert len(value) == b and len(policy) > b and len(pre_value) == b           # every root starts a street here
    assert float(value.value_targets.abs().max()) <= 1.0                         # clamped (cfr_evaluator.py:1394)
    assert torch.isfinite(pre_value.value_targets).all()                         # chance-node means: not clamped there
    pt = policy.policy_targets
    assert pt.shape[1:] == (H, 5) and not pt.permute(0, 2, 1)[~policy.legal_masks].any()
    mass = pt.sum(-1)
    assert ((mass - 1).abs() < 1e-4).logical_or(mass.abs() < 1e-6).all()          # a distribution, or a blocked hand
    del value, pre_value, policy, pt, mass, ev, nxt
    torch.cuda.empty_cache()
    # batch independence with the network in fp32 (bf16 results depend on the GEMM tiling too much to compare)
    big, _ = run(b, None)
    ref, _ = run(small, None)
    rows = rows_of_first_roots(big, small)
    assert len(rows) == ref.total_nodes
    rows = torch.from_numpy(rows).to(DEV)
    for name in ("policy_probs_avg", "beliefs_avg", "values_avg"):
        same_but_few(getattr(big, name)[rows], getattr(ref, name), name)
    del big, ref
    torch.cuda.empty_cache()
    # and bit for bit with a network that has no GEMM in it (see the turn test above); the sampled policy is a
    # snapshot at an iteration drawn per root from the generator, whose draws depend on the batch
    big, _ = run(b, None, 6, RowWiseNetwork())
    ref, _ = run(small, None, 6, RowWiseNetwork())
    for name in STATE_TENSORS:
        if name == "policy_probs_sample":
            continue
        assert torch.equal(getattr(big, name)[rows], getattr(ref, name)), name


def test_generator_with_the_reference_production_settings():
    """The self-play loop with every search setting of the reference's own configuration
    (conf/config_rebel_cfr.yaml: 192 hands, blinds 5 / 10 at 100 big blinds, bins 0.5 / 1 pot,
    depth 5, discounted_plus with delay, `model` warm start x 10, alpha 2->4 / beta -1->-2 /
    gamma 5->0 schedules, value targets from the final average strategy, a zero-sum network),
    iterations scaled down from 200 / 15 / 80 to 16 / 3 / 6.  Properties only: the loop runs for
    several passes, hands advance and are replaced, every batch is finite and in range."""
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.fused_cfr_hip import CFRType
    from poker2_amd.leaf_models import NetworkLeafModel, RangeBoardMLP
    from poker2_amd.rebel_data_generator import EnvProto, RebelDataGenerator
    n = 192
    dev = torch.device(DEV)
    cfg = river_dcfr_config(n, iterations=16, depth=5, dcfr_delay=6)
    z = cfg.search
    z.cfr_type, z.cfr_plus, z.cfr_avg = CFRType.discounted_plus, False, False
    z.warm_start_iterations, z.warm_start_type, z.warm_start_multiplier = 3, "model", 10.0
    z.dcfr_alpha, z.dcfr_alpha_final, z.dcfr_beta, z.dcfr_beta_final = 2.0, 4.0, -1.0, -2.0
    z.dcfr_gamma, z.dcfr_gamma_final = 5.0, 0.0
    z.value_targets_from_final_policy = True
    cfg.env.bet_bins, cfg.env.bb = [0.5, 1.0], 10
    env_gen = torch.Generator(device="cpu")
    env_gen.manual_seed(3)
    search_gen = torch.Generator(device=dev)
    search_gen.manual_seed(4)
    net = RangeBoardMLP(hidden=256, layers=2).to(dev)
    model = NetworkLeafModel(net, dev, enforce_zero_sum=True, autocast_dtype=torch.bfloat16)
    ev = HipSparseCFREvaluator(model, dev, cfg, generator=search_gen)

    class Buffer:
        def __init__(self):
            self.batches = []

        def add_batch(self, batch):
            self.batches.append(batch)
    value_buffer, policy_buffer = Buffer(), Buffer()
    dg = RebelDataGenerator(EnvProto(mean_stack=1000, sb=5, bb=10, randomize_stacks=True, rng=env_gen), ev,
                            value_buffer, policy_buffer)
    assert (dg.current_pbs.env.pot == 15).all() and (dg.current_pbs.env.min_raise == 10).all()
    streets_seen = set()
    for _ in range(3):
        value_batch, policy_batch = dg.generate_data(300)
        assert len(value_batch) >= 300 - n and len(policy_batch) > 0
        streets_seen |= set(np.asarray(dg.current_pbs.env.street).tolist())
    passes = len(policy_buffer.batches)
    assert passes >= 4 and len(value_buffer.batches) == 2 * passes
    assert len(streets_seen) >= 2                                        # hands moved on to later streets
    for i, b in enumerate(value_buffer.batches):
        if len(b) == 0:
            continue
        vt = b.value_targets
        assert torch.isfinite(vt).all() and torch.isfinite(b.features.beliefs).all()
        if i % 2 == 0:
            assert float(vt.abs().max()) <= 1.0                          # the clamped batch
        s = b.features.beliefs.view(len(b), 2, H).sum(-1)
        torch.testing.assert_close(s, torch.ones_like(s), rtol=0, atol=1e-4)
    for b in policy_buffer.batches:
        pt = b.policy_targets
        assert torch.isfinite(pt).all() and not pt.permute(0, 2, 1)[~b.legal_masks].any()
        mass = pt.sum(-1)
        assert ((mass - 1).abs() < 1e-4).logical_or(mass.abs() < 1e-6).all()
