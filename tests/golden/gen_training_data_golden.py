"""Writes tests/golden/training_data_golden.npz by RUNNING the reference's own
``SparseCFREvaluator`` (search, ``training_data``: src/p2/search/cfr_evaluator.py:1383-1495) with
its ``RebelFeatureEncoder`` (src/p2/models/mlp/rebel_feature_encoder.py:55-127) and
``ChanceNodeHelper`` on the CPU of the build container.  Run once, here only:
    python tests/golden/gen_training_data_golden.py

Roots come from playing the reference env forward from its reset state with scripted bins, so
every field (committed chips, previous board, min raise) is what the env itself produces: turn
and river and flop roots at the start of a betting round (these get pre-chance value targets
through the single-card / flop chance node), roots in the middle of a round, preflop roots (the
reset state is dropped from the value batch).  The leaf network is a closed-form function of the
encoded features (written out in ``ValueNet`` below; tests restate it), so the search, the
encoder and the chance nodes all feed the stored targets.  Two more cases use the reference's default algorithm (linear CFR with
CFR+, cfr_avg, zero-sum network; with and without the warm start).  A last case has the shape of
the reference's production settings (discounted_plus with delay, model warm start, alpha / beta /
gamma schedules, value targets from the final average strategy).  The flop chance node runs in its
exhaustive mode (all classes, all 24 permutations): nothing is drawn at random.
Each case also holds one whole ``evaluate_cfr`` (sampling schedule, search, leaf sampling with
exploration and dealing) run from a CPU generator seeded 77: the iterations it snapshots and the
leaves it returns.  A last section holds what the env's ``reset`` deals from a seeded CPU generator.

With ``--fused`` the same searches run through the reference's ``FusedSparseCFREvaluator``, its
Triton kernels executing under Triton's CPU interpreter, and go to
``fused_training_data_golden.npz`` (how, and why ``-O``: see gen_cfr_golden.py):
    python -O tests/golden/gen_training_data_golden.py --fused
"""
from __future__ import annotations

import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from gen_cfr_golden import REF_SRC, install_stand_ins  # noqa: E402

ENV_FIELDS = ("street", "to_act", "button", "pot", "stacks", "committed", "min_raise", "actions_this_round",
              "is_allin", "starting_stacks", "scale", "board_indices", "last_board_indices", "done")
STATE = ("policy_probs_avg", "beliefs", "beliefs_avg", "values_avg")

# name, depth, last iteration + 1, per root: (button, bins played from the reset state), search settings
DEFAULTS = {"cfr_type": "discounted", "cfr_plus": False, "cfr_avg": False, "warm": 0, "enforce_zero_sum": False,
            "delay": 0, "alpha": 1.5, "beta": 0.0, "gamma": 2.0, "alpha_final": None, "beta_final": None,
            "gamma_final": None, "warm_type": "model_br", "warm_mult": 1.0, "final_policy_values": False,
            "base_only": False}
DISCOUNTED = {}
CASES = [
    ("streets_mixed", 3, 4, [(0, [1, 1, 1, 1]), (1, [3, 1, 1, 1]), (0, [1, 1, 1, 1, 1, 1]),
                             (1, [1, 1, 1, 1, 1, 1, 2]), (0, [2, 1]), (1, [1, 1, 1, 1, 1])], DISCOUNTED),
    ("preflop", 2, 3, [(0, []), (1, [1]), (1, [])], DISCOUNTED),
    # the reference's default algorithm (structured_config.py:236-265: linear CFR with CFR+, leaf values
    # de-averaged for cfr_avg, a model_br warm start) with a network that asks for zero-sum values
    ("linear_avg_zero_sum", 3, 5, [(0, [1, 1, 1, 1]), (1, [1, 1, 1, 1, 1, 1]), (0, [1, 1, 1, 1, 2]), (1, [2, 1])],
     {"cfr_type": "linear", "cfr_plus": True, "cfr_avg": True, "warm": 0, "enforce_zero_sum": True}),
    # the same with the warm start; base class only: the fused class runs its warm start with device scalars that
    # no iteration has filled yet (see gen_cfr_golden.py), which under linear CFR also feeds the leaf de-averaging
    ("linear_avg_zero_sum_warm", 3, 6, [(0, [1, 1, 1, 1]), (1, [1, 1, 1, 1, 1, 1]), (0, [1, 1, 1, 1, 2]), (1, [2, 1])],
     {"cfr_type": "linear", "cfr_plus": True, "cfr_avg": True, "warm": 2, "enforce_zero_sum": True, "base_only": True}),
    # the shape of the reference's own search settings (conf/config_rebel_cfr.yaml:70-92), scaled down: discounted_plus
    # with a delay that outlasts the warm start, `model` warm start x 10, alpha / beta / gamma schedules towards their
    # `_final` values, value targets taken from the final average strategy
    ("production_like", 3, 9, [(1, [1, 1, 1, 1]), (0, [1, 1, 1, 1, 1, 1]), (1, [1, 1, 1, 1, 2]), (0, [1, 1, 3, 1])],
     {"cfr_type": "discounted_plus", "delay": 4, "warm": 3, "warm_type": "model", "warm_mult": 10.0, "alpha": 2.0,
      "alpha_final": 4.0, "beta": -1.0, "beta_final": -2.0, "gamma": 5.0, "gamma_final": 0.0,
      "final_policy_values": True}),
]


def main(fused: bool = False) -> None:
    os.environ.setdefault("TORCHDYNAMO_DISABLE", "1")
    if fused:
        if __debug__:
            raise SystemExit("run as: python -O tests/golden/gen_training_data_golden.py --fused")
        os.environ["TRITON_INTERPRET"] = "1"          # before triton is imported
    install_stand_ins()
    sys.path.insert(0, REF_SRC)
    import warnings
    import torch
    from p2.core.structured_config import (CFRType, Config, EnvConfig, ModelConfig, SearchConfig, TrainingConfig,
                                           WarmStartType)
    from p2.env.card_utils import NUM_HANDS
    from p2.env.hunl_tensor_env import HUNLTensorEnv
    from p2.models.model_output import ModelOutput
    from p2.models.mlp.rebel_feature_encoder import RebelFeatureEncoder
    from p2.search.sparse_cfr_evaluator import SparseCFREvaluator
    if fused:
        from p2.search.fused_sparse_cfr_evaluator import FusedSparseCFREvaluator
    warnings.filterwarnings("ignore")

    class ValueNet:
        """hand value of player p, hand h =
             s_p * 0.05 * w * (1326 * opponent_range[h] - 1) + 0.002 * ((h mod 7) - 3)
        with s_0 = 1, s_1 = -1 and
             w = 0.2 + 0.1 * context[2] + 0.05 * context[1] - 0.03 * context[3]
                 + 0.01 / 13 * sum over dealt board cards of (rank + 1)."""

        def __init__(self, num_actions, enforce_zero_sum=False):
            self.num_actions = num_actions
            self.enforce_zero_sum = enforce_zero_sum
            self.hidden_dim = 1

        def create_feature_encoder(self, env, device=None, dtype=None):
            return RebelFeatureEncoder(env=env, device=device, dtype=dtype)

        def eval(self):
            pass

        def __call__(self, f, include_policy=True):
            b = f.beliefs.view(-1, 2, NUM_HANDS).float()
            ranks = torch.where(f.board >= 0, (f.board % 13 + 1).float(), torch.zeros_like(f.board, dtype=torch.float32))
            w = (0.2 + 0.1 * f.context[:, 2] + 0.05 * f.context[:, 1] - 0.03 * f.context[:, 3]
                 + 0.01 / 13.0 * ranks.sum(dim=1))
            opp = torch.flip(b, dims=[1])
            sign = torch.tensor([1.0, -1.0])[None, :, None]
            h = ((torch.arange(NUM_HANDS) % 7).float() - 3.0) * 0.002
            hv = sign * 0.05 * w[:, None, None] * (NUM_HANDS * opp - 1.0) + h[None, None, :]
            return ModelOutput(policy_logits=torch.zeros(b.shape[0], NUM_HANDS, self.num_actions),
                               value=torch.zeros(b.shape[0]), hand_values=hv)

    rng = np.random.default_rng(515)
    cols = np.sort(rng.choice(NUM_HANDS, 64, replace=False))
    cases = [c for c in CASES if not (fused and c[4].get("base_only", False))]
    out = {"columns": cols, "case_names": np.array([c[0] for c in cases])}
    dev = torch.device("cpu")
    bins = [0.5, 1.0]
    for name, depth, iters, scripts, overrides in cases:
        algo = {**DEFAULTS, **overrides}
        n = len(scripts)
        env = HUNLTensorEnv(num_envs=n, starting_stack=1000, sb=50, bb=100, default_bet_bins=list(bins), device=dev)
        deck = torch.stack([torch.from_numpy(rng.permutation(52)[:9].copy()) for _ in range(n)])
        env.reset(force_button=torch.tensor([s[0] for s in scripts]), force_deck=deck)
        for step in range(max(len(s[1]) for s in scripts)):
            env.step_bins(torch.tensor([s[1][step] if step < len(s[1]) else -1 for s in scripts], dtype=torch.long))
        assert not env.done.any()

        cfg = Config()
        cfg.device = "cpu"
        cfg.num_envs = n
        cfg.train = TrainingConfig()
        cfg.model = ModelConfig()
        cfg.model.num_actions = len(bins) + 3
        cfg.env = EnvConfig()
        cfg.env.stack, cfg.env.sb, cfg.env.bb, cfg.env.bet_bins, cfg.env.flop_showdown = 1000, 50, 100, bins, False
        cfg.search = SearchConfig()
        cfg.search.iterations = iters
        cfg.search.warm_start_iterations = algo["warm"]
        cfg.search.depth = depth
        cfg.search.dcfr_alpha, cfg.search.dcfr_beta, cfg.search.dcfr_gamma = algo["alpha"], algo["beta"], algo["gamma"]
        cfg.search.dcfr_alpha_final, cfg.search.dcfr_beta_final = algo["alpha_final"], algo["beta_final"]
        cfg.search.dcfr_gamma_final = algo["gamma_final"]
        cfg.search.dcfr_plus_delay = algo["delay"]
        cfg.search.warm_start_type = WarmStartType[algo["warm_type"]]
        cfg.search.warm_start_multiplier = algo["warm_mult"]
        cfg.search.value_targets_from_final_policy = algo["final_policy_values"]
        cfg.search.cfr_type = CFRType[algo["cfr_type"]]
        cfg.search.cfr_plus = algo["cfr_plus"]
        cfg.search.cfr_avg = algo["cfr_avg"]
        ev = SparseCFREvaluator(model=ValueNet(len(bins) + 3, algo["enforce_zero_sum"]), device=dev, cfg=cfg)
        if fused:
            ev.__class__ = FusedSparseCFREvaluator
            ev._ensure_fused_attrs()
        ev.chance_helper.FLOP_SAMPLE_SIZE = 0
        ev.chance_helper.NUM_PERM_SAMPLES = 0

        bel = rng.gamma(0.5, size=(n, 2, NUM_HANDS)).astype(np.float32)
        bel /= bel.sum(-1, keepdims=True)
        for f in ENV_FIELDS:
            out[f"{name}/root/{f}"] = getattr(env, f).clone().numpy()
        ev.initialize_subgame(env, torch.arange(n), initial_beliefs=torch.from_numpy(bel.copy()))
        ev.initialize_policy_and_beliefs()               # evaluate_cfr (cfr_evaluator.py:1497-1518) without its draws
        if algo["warm"] > 0:
            ev.warm_start()
        ev.set_leaf_values(0)
        ev.compute_expected_values()
        ev.values_avg[:] = ev.latest_values
        ev.t_sample = torch.full((ev.total_nodes,), -1, dtype=torch.long)
        for t in range(algo["warm"], iters):
            ev.cfr_iteration(t)
        if ev.use_final_policy_values:
            ev.update_average_values_final()
        for s in STATE:
            x = getattr(ev, s).detach().numpy()
            out[f"{name}/state/{s}"] = np.ascontiguousarray(x[..., cols]).astype(np.float32)
            out[f"{name}/state/{s}_rowsum"] = x.astype(np.float64).sum(-1)
        # the encoder alone, on every node, with the leaf rule for the board (cfr_evaluator.py:1031-1033)
        enc = ev.feature_encoder.encode(ev.beliefs, pre_chance_node=ev.new_street_mask)
        out[f"{name}/encode_leaf/context"] = enc.context.numpy()
        out[f"{name}/encode_leaf/board"] = enc.board.numpy()
        out[f"{name}/encode_leaf/to_act"] = enc.to_act.numpy()
        out[f"{name}/encode_leaf/street"] = enc.street.numpy()
        out[f"{name}/new_street_mask"] = ev.new_street_mask.numpy()
        out[f"{name}/leaf_mask"] = ev.leaf_mask.numpy()

        batches = dict(zip(("value", "pre_value", "policy"), ev.training_data()))
        for tag, batch in batches.items():
            p = f"{name}/{tag}"
            out[f"{p}/len"] = np.int64(len(batch))
            out[f"{p}/context"] = batch.features.context.numpy()
            out[f"{p}/board"] = batch.features.board.numpy()
            out[f"{p}/to_act"] = batch.features.to_act.numpy()
            out[f"{p}/street"] = batch.features.street.numpy()
            fb = batch.features.beliefs.numpy().reshape(-1, 2, NUM_HANDS)
            out[f"{p}/beliefs"] = np.ascontiguousarray(fb[..., cols])
            out[f"{p}/beliefs_rowsum"] = fb.astype(np.float64).sum(-1)
            out[f"{p}/legal_masks"] = batch.legal_masks.numpy()
            if batch.value_targets is not None:
                out[f"{p}/value_targets"] = batch.value_targets.numpy().astype(np.float32)
            if batch.policy_targets is not None:
                pt = batch.policy_targets.numpy()
                out[f"{p}/policy_targets"] = np.ascontiguousarray(pt[:, cols, :]).astype(np.float32)
                out[f"{p}/policy_targets_sum"] = pt.astype(np.float64).sum(axis=1)
            for k, v in batch.statistics.items():
                out[f"{p}/stat/{k}"] = v.numpy()
        # the whole search with its random parts (cfr_evaluator.py:1497-1528: sampling schedule, search, leaf
        # sampling with exploration, sparse_cfr_evaluator.py:325-426) from a seeded CPU generator
        gen = torch.Generator(device="cpu")
        gen.manual_seed(77)
        ev2 = SparseCFREvaluator(model=ValueNet(len(bins) + 3, algo["enforce_zero_sum"]), device=dev, cfg=cfg,
                                 generator=gen)
        if fused:
            ev2.__class__ = FusedSparseCFREvaluator
            ev2._ensure_fused_attrs()
        ev2.initialize_subgame(env, torch.arange(n), initial_beliefs=torch.from_numpy(bel.copy()))
        pbs = ev2.evaluate_cfr(training_mode=True)
        out[f"{name}/search/seed"] = np.int64(77)
        out[f"{name}/search/root_deck"] = env.deck.clone().numpy()
        out[f"{name}/search/t_sample"] = ev2.t_sample.numpy()
        for f in ENV_FIELDS + ("deck",):
            out[f"{name}/search/leaf/{f}"] = getattr(pbs.env, f).clone().numpy()
        lb = pbs.beliefs.numpy()
        out[f"{name}/search/leaf_beliefs"] = np.ascontiguousarray(lb[..., cols]).astype(np.float32)
        out[f"{name}/search/leaf_beliefs_rowsum"] = lb.astype(np.float64).sum(-1)
        print(name, "sampled leaves", lb.shape[0], "streets", getattr(pbs.env, "street").tolist(), flush=True)
        out[f"{name}/beliefs"] = bel
        out[f"{name}/depth_offsets"] = np.array(ev.depth_offsets, dtype=np.int64)
        out[f"{name}/settings"] = np.array([str(depth), str(iters), json.dumps(algo)])
        print(name, "nodes", ev.total_nodes, "depth offsets", ev.depth_offsets,
              {k: len(b) for k, b in batches.items()}, flush=True)
    # the env's own reset (hunl_tensor_env.py:219-346) from a seeded CPU generator: button, deck, stacks
    gen = torch.Generator(device="cpu")
    gen.manual_seed(99)
    env = HUNLTensorEnv(num_envs=16, mean_stack=1000, sb=50, bb=100, default_bet_bins=list(bins), device=dev, rng=gen,
                        randomize_stacks=True)
    env.reset()
    for f in ENV_FIELDS + ("deck",):
        out[f"reset/{f}"] = getattr(env, f).clone().numpy()
    out["reset/seed"] = np.int64(99)
    path = os.path.join(HERE, "fused_training_data_golden.npz" if fused else "training_data_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path) // 1024, "KiB")


if __name__ == "__main__":
    main(fused="--fused" in sys.argv[1:])
