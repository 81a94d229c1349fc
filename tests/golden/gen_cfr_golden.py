"""Writes tests/golden/cfr_golden.npz by RUNNING the reference's own ``SparseCFREvaluator``
(the torch base path of the search, CPU) in the build container.  Run once, here only:

    python tests/golden/gen_cfr_golden.py

Nothing else in the reference pins multi-iteration CFR numbers (its evaluator tests are
structural), so these vectors are what ties the oracle's whole iteration to the reference.
``p2.core.structured_config`` imports hydra / omegaconf at module top only to register the
config dataclass; they are absent here, so two empty stand-in modules are placed in
``sys.modules`` before the import (``ConfigStore.instance().store`` becomes a no-op; no
arithmetic goes through them).  torch.compile is switched off (TORCHDYNAMO_DISABLE) so the
showdown evaluation runs eagerly.

Cases: river roots (so showdown leaves, fold leaves and depth-limited model leaves all occur),
zero-value / uniform-policy mock network like the reference's own ``MockModel``
(tests/test_sparse_cfr_evaluator.py:43-86), seeded Dirichlet ranges.  The fixture stores the
inputs (boards, ranges, chips, settings), the tree arrays, and after the preparation step and
the first two iterations, the sampling iteration and the last one, the 11 state tensors
restricted to 64 seeded hand columns plus their full row sums (float64).  Two cases start from
the reference's warm start (``model_br`` and ``model``).

With ``--fused`` the same searches run through the reference's ``FusedSparseCFREvaluator`` (the
class the search path uses on a GPU) and go to ``fused_cfr_golden.npz``:

    python -O tests/golden/gen_cfr_golden.py --fused

Its Triton kernels execute on CPU tensors under Triton's interpreter (TRITON_INTERPRET=1).  The
evaluator is built as a ``SparseCFREvaluator`` and its ``__class__`` is then set to the fused
class and ``_ensure_fused_attrs()`` called, which is how the reference's own tests construct it
(tests/test_fused_cfr_triton.py:600, 646-647); the hand ranker therefore stays ``rules.py``.
``-O`` is needed because one wrapper guards its launch with ``assert target.is_cuda``
(fused_cfr_triton.py:307).

In the fused fixture the case ``warm_model_d2`` holds NaN in ``policy_probs_avg`` and what derives
from it: the fused class mixes the average policy with the device scalars of ``TScalars``, which are
still all zero when ``warm_start`` calls ``update_policy`` before the first ``cfr_iteration``
(fused_sparse_cfr_evaluator.py:368-378, fused_cfr_triton.py:2109-2128), unless the discount delay
sends that call down the copy branch (:356-361) as the reference's own settings do.
"""
from __future__ import annotations

import os
import sys
import types

import numpy as np

REF_SRC = "/root/reference/src"
HERE = os.path.dirname(os.path.abspath(__file__))
STATE = ("policy_probs", "policy_probs_avg", "policy_probs_sample", "cumulative_regrets", "regret_weight_sums",
         "self_reach", "self_reach_avg", "beliefs", "beliefs_avg", "latest_values", "values_avg")

# name, cfr_type, cfr_plus, cfr_avg, dcfr_plus_delay, depth, last iteration + 1,
# rows of (pot, stack0, stack1, button), (warm_start_iterations, warm_start_type, warm_start_multiplier)
CASES = [
    ("discounted_d2", "discounted", False, False, 0, 2, 6, [(200, 800, 800, 0), (200, 800, 800, 1)], (0, "model_br", 1.0)),
    ("dplus_d3", "discounted_plus", False, False, 2, 3, 6, [(300, 500, 900, 1), (120, 2000, 700, 0)], (0, "model_br", 1.0)),
    ("linear_avg_d2", "linear", True, True, 0, 2, 5, [(200, 800, 800, 0)], (0, "model_br", 1.0)),
    ("linear_noplus_d2", "linear", False, True, 0, 2, 5, [(200, 800, 800, 1)], (0, "model_br", 1.0)),
    ("standard_d2", "standard", False, False, 0, 2, 4, [(450, 300, 300, 1)], (0, "model_br", 1.0)),
    ("warm_br_d2", "discounted_plus", False, False, 4, 2, 7, [(200, 800, 800, 1)], (3, "model_br", 1.0)),
    ("warm_model_d2", "discounted", False, False, 0, 2, 6, [(260, 700, 900, 0)], (3, "model", 10.0)),
    # the shape of the reference's own search settings (conf/config_rebel_cfr.yaml:77-86): model warm start under
    # discounted_plus with a delay that outlasts the warm start iterations
    ("warm_model_dplus_d2", "discounted_plus", False, False, 5, 2, 8, [(240, 900, 650, 1)], (3, "model", 10.0)),
]


def install_stand_ins() -> None:
    hydra = types.ModuleType("hydra")
    core = types.ModuleType("hydra.core")
    store = types.ModuleType("hydra.core.config_store")

    class ConfigStore:
        @classmethod
        def instance(cls):
            return cls()

        def store(self, *a, **k):
            return None
    store.ConfigStore = ConfigStore
    hydra.core = core
    core.config_store = store
    omega = types.ModuleType("omegaconf")

    class DictConfig(dict):
        pass

    class OmegaConf:
        @staticmethod
        def to_container(cfg, **k):
            return dict(cfg)
    omega.DictConfig = DictConfig
    omega.OmegaConf = OmegaConf
    sys.modules.update({"hydra": hydra, "hydra.core": core, "hydra.core.config_store": store, "omegaconf": omega})


def main(fused: bool = False) -> None:
    os.environ.setdefault("TORCHDYNAMO_DISABLE", "1")
    if fused:
        if __debug__:
            raise SystemExit("run as: python -O tests/golden/gen_cfr_golden.py --fused")
        os.environ["TRITON_INTERPRET"] = "1"          # before triton is imported
    install_stand_ins()
    sys.path.insert(0, REF_SRC)
    import torch
    from p2.core.structured_config import (CFRType, Config, EnvConfig, ModelConfig, SearchConfig, TrainingConfig,
                                           WarmStartType)
    from p2.env.card_utils import NUM_HANDS
    from p2.env.hunl_tensor_env import HUNLTensorEnv
    from p2.models.model_output import ModelOutput
    from p2.search.sparse_cfr_evaluator import SparseCFREvaluator
    if fused:
        from p2.search.fused_sparse_cfr_evaluator import FusedSparseCFREvaluator

    class MockModel:
        def __init__(self, num_actions):
            self.num_actions = num_actions
            self.enforce_zero_sum = True
            self.hidden_dim = 1

        def create_feature_encoder(self, env, device=None, dtype=None):
            from p2.models.mlp.rebel_feature_encoder import RebelFeatureEncoder
            return RebelFeatureEncoder(env=env, device=device, dtype=dtype)

        def __call__(self, features, include_policy=True):
            b = len(features)
            return ModelOutput(policy_logits=torch.zeros(b, NUM_HANDS, self.num_actions),
                               value=torch.zeros(b), hand_values=torch.zeros(b, 2, NUM_HANDS))

        def eval(self):
            pass

    rng = np.random.default_rng(2024)
    cols = np.sort(rng.choice(NUM_HANDS, 64, replace=False))
    out = {"columns": cols, "case_names": np.array([c[0] for c in CASES])}
    dev = torch.device("cpu")
    for name, cfr_type, cfr_plus, cfr_avg, delay, depth, iters, rows, (warm, warm_type, warm_mult) in CASES:
        n = len(rows)
        bins = [0.5, 1.0]
        env = HUNLTensorEnv(num_envs=n, starting_stack=1000, sb=50, bb=100, default_bet_bins=list(bins), device=dev)
        deck = torch.stack([torch.from_numpy(rng.permutation(52)[:9].copy()) for _ in range(n)])
        env.reset(force_button=torch.tensor([r[3] for r in rows]), force_deck=deck)
        for _ in range(6):
            env.step_bins(torch.ones(n, dtype=torch.long))
        assert (env.street == 3).all() and (env.actions_this_round == 0).all()
        pot = torch.tensor([r[0] for r in rows])
        stacks = torch.tensor([[r[1], r[2]] for r in rows])
        env.pot[:] = pot
        env.stacks[:] = stacks
        env.starting_stacks[:] = stacks + (pot // 2)[:, None]
        env.scale[:] = env.starting_stacks[:, 0].float()

        cfg = Config()
        cfg.device = "cpu"
        cfg.num_envs = n
        cfg.train = TrainingConfig()
        cfg.model = ModelConfig()
        cfg.model.num_actions = len(bins) + 3
        cfg.env = EnvConfig()
        cfg.env.stack, cfg.env.sb, cfg.env.bb, cfg.env.bet_bins, cfg.env.flop_showdown = 1000, 50, 100, bins, False
        cfg.search = SearchConfig()
        cfg.search.iterations = 50
        cfg.search.warm_start_iterations = warm
        cfg.search.warm_start_type = WarmStartType[warm_type]
        cfg.search.warm_start_multiplier = warm_mult
        cfg.search.depth = depth
        cfg.search.dcfr_alpha, cfg.search.dcfr_beta, cfg.search.dcfr_gamma = 1.5, 0.0, 2.0
        cfg.search.dcfr_plus_delay = delay
        cfg.search.cfr_type = CFRType[cfr_type]
        cfg.search.cfr_plus = cfr_plus
        cfg.search.cfr_avg = cfr_avg
        ev = SparseCFREvaluator(model=MockModel(len(bins) + 3), device=dev, cfg=cfg)
        if fused:
            ev.__class__ = FusedSparseCFREvaluator
            ev._ensure_fused_attrs()                                  # as tests/test_fused_cfr_triton.py:646-647 does

        board = env.board_indices.clone().numpy()
        bel = rng.gamma(0.5, size=(n, 2, NUM_HANDS)).astype(np.float32)
        bel /= bel.sum(-1, keepdims=True)
        ev.initialize_subgame(env, torch.arange(n), initial_beliefs=torch.from_numpy(bel.copy()))
        # evaluate_cfr without the random sampling schedule and the leaf sampling (:1497-1528)
        ev.initialize_policy_and_beliefs()
        if warm > 0:
            ev.warm_start()
        ev.set_leaf_values(0)
        ev.compute_expected_values()
        ev.values_avg[:] = ev.latest_values
        ev.t_sample = torch.full((ev.total_nodes,), -1, dtype=torch.long)
        ev.t_sample[ev._fan_out_deep(torch.arange(n)) == 0] = 2      # root 0 samples its policy at t = 2

        def snap(tag):
            for s in STATE:
                x = getattr(ev, s).detach().numpy()
                out[f"{name}/{tag}/{s}"] = np.ascontiguousarray(x[..., cols]).astype(np.float32)
                out[f"{name}/{tag}/{s}_rowsum"] = x.astype(np.float64).sum(-1)
        snap("prep")
        stored = []
        for t in range(warm, iters):
            ev.cfr_iteration(t)
            if t in (warm, warm + 1, 2, iters - 1):     # first two, the sampling iteration, the last
                snap(f"t{t}")
                stored.append(t)
        out[f"{name}/stored"] = np.array(stored, dtype=np.int64)
        stats = ev._compute_exploitability()                 # cfr_evaluator.py:718-764
        out[f"{name}/local_exploitability"] = stats.local_exploitability.numpy().astype(np.float32)
        out[f"{name}/local_best_response_values"] = stats.local_best_response_values.numpy().astype(np.float32)
        out[f"{name}/board"] = board
        out[f"{name}/beliefs"] = bel
        out[f"{name}/rows"] = np.array(rows, dtype=np.int64)
        out[f"{name}/depth_offsets"] = np.array(ev.depth_offsets, dtype=np.int64)
        for s in ("parent_index", "action_from_parent", "child_count", "child_offsets", "prev_actor"):
            out[f"{name}/{s}"] = getattr(ev, s).numpy().astype(np.int64)
        out[f"{name}/to_act"] = ev.env.to_act.numpy().astype(np.int64)
        out[f"{name}/settings"] = np.array([cfr_type, str(cfr_plus), str(cfr_avg), str(delay), str(depth), str(iters),
                                            str(warm), warm_type, str(warm_mult)])
        print(name, "nodes", ev.total_nodes, "depth offsets", ev.depth_offsets, flush=True)
    path = os.path.join(HERE, "fused_cfr_golden.npz" if fused else "cfr_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path) // 1024, "KiB")


if __name__ == "__main__":
    main(fused="--fused" in sys.argv[1:])
