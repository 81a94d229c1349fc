"""Writes tests/golden/generator_golden.npz by RUNNING the reference's own self-play loop —
``RebelDataGenerator.generate_data`` (src/p2/search/rebel_data_generator.py:11-95) around its
``SparseCFREvaluator`` and ``HUNLTensorEnv`` — on the CPU of the build container.  Run once, here
only:
    python tests/golden/gen_generator_golden.py

Two seeded CPU generators carry every random choice: the env's (button, deck and stacks of each
reset, hunl_tensor_env.py:219-346) and the evaluator's (sampling schedule, leaf walk, flop classes
and suit permutations of the flop chance node).  The hands start at the reset state with uniform
ranges; the loop searches them, stores training batches, continues from the sampled leaves and
deals fresh hands into the freed slots, until the asked number of value samples exists.  The
leaf network is the closed form of gen_training_data_golden.py.  The fixture holds what each
pass of the loop handed to the buffers, what the call returned, and the states it left behind.

With ``--fused`` the evaluator is the reference's ``FusedSparseCFREvaluator`` with its Triton kernels
under Triton's CPU interpreter (how, and why ``-O``: see gen_cfr_golden.py); output goes to
``fused_generator_golden.npz``:
    python -O tests/golden/gen_generator_golden.py --fused
One thing is changed in that run.  The fused class keeps ``root_index`` (the root of every node)
in a cache that is keyed by the node count alone (fused_sparse_cfr_evaluator.py:124-138).  The
generator reuses one evaluator for every subgame, and two consecutive subgames here have the same
node count but different trees, so from the second on the beliefs of deep nodes are taken from the
wrong roots: with the cache left alone this run's value targets differ from the base class's by
up to 3e-2 on two states of the fifth pass; with it cleared before each ``initialize_subgame`` the
two classes agree to 7e-6.  The fixture is written with the cache cleared, i.e. it states what the
class computes on a fresh object.
"""
from __future__ import annotations

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from gen_cfr_golden import REF_SRC, install_stand_ins  # noqa: E402

ENV_FIELDS = ("street", "to_act", "button", "pot", "stacks", "committed", "min_raise", "actions_this_round",
              "is_allin", "starting_stacks", "scale", "board_indices", "last_board_indices", "done", "deck")
N_ENVS, DEPTH, ITERATIONS, ASKED = 6, 2, 3, 40
ENV_SEED, SEARCH_SEED = 2024, 4048


def main(fused: bool = False) -> None:
    os.environ.setdefault("TORCHDYNAMO_DISABLE", "1")
    if fused:
        if __debug__:
            raise SystemExit("run as: python -O tests/golden/gen_generator_golden.py --fused")
        os.environ["TRITON_INTERPRET"] = "1"          # before triton is imported
    install_stand_ins()
    sys.path.insert(0, REF_SRC)
    import warnings
    import torch
    from p2.core.structured_config import CFRType, Config, EnvConfig, ModelConfig, SearchConfig, TrainingConfig
    from p2.env.card_utils import NUM_HANDS
    from p2.env.hunl_tensor_env import HUNLTensorEnv
    from p2.models.model_output import ModelOutput
    from p2.models.mlp.rebel_feature_encoder import RebelFeatureEncoder
    from p2.search.rebel_data_generator import RebelDataGenerator
    from p2.search.sparse_cfr_evaluator import SparseCFREvaluator
    warnings.filterwarnings("ignore")

    class ValueNet:          # the closed form documented in gen_training_data_golden.py
        def __init__(self, num_actions):
            self.num_actions = num_actions
            self.enforce_zero_sum = False
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

    rng = np.random.default_rng(616)
    cols = np.sort(rng.choice(NUM_HANDS, 64, replace=False))
    out = {"columns": cols, "settings": np.array([N_ENVS, DEPTH, ITERATIONS, ASKED, ENV_SEED, SEARCH_SEED], dtype=np.int64)}
    dev = torch.device("cpu")
    bins = [0.5, 1.0]
    env_gen = torch.Generator(device="cpu")
    env_gen.manual_seed(ENV_SEED)
    search_gen = torch.Generator(device="cpu")
    search_gen.manual_seed(SEARCH_SEED)
    env_proto = HUNLTensorEnv(num_envs=N_ENVS, mean_stack=1000, sb=50, bb=100, default_bet_bins=list(bins), device=dev,
                              rng=env_gen, randomize_stacks=True)
    cfg = Config()
    cfg.device = "cpu"
    cfg.num_envs = N_ENVS
    cfg.train = TrainingConfig()
    cfg.model = ModelConfig()
    cfg.model.num_actions = len(bins) + 3
    cfg.env = EnvConfig()
    cfg.env.stack, cfg.env.sb, cfg.env.bb, cfg.env.bet_bins, cfg.env.flop_showdown = 1000, 50, 100, bins, False
    cfg.search = SearchConfig()
    cfg.search.iterations = ITERATIONS
    cfg.search.warm_start_iterations = 0
    cfg.search.depth = DEPTH
    cfg.search.dcfr_alpha, cfg.search.dcfr_beta, cfg.search.dcfr_gamma = 1.5, 0.0, 2.0
    cfg.search.dcfr_plus_delay = 0
    cfg.search.cfr_type = CFRType["discounted"]
    cfg.search.cfr_plus = False
    cfg.search.cfr_avg = False
    ev = SparseCFREvaluator(model=ValueNet(len(bins) + 3), device=dev, cfg=cfg, generator=search_gen)
    if fused:
        from p2.search.fused_sparse_cfr_evaluator import FusedSparseCFREvaluator

        class FreshRootIndex(FusedSparseCFREvaluator):
            def initialize_subgame(self, *args, **kwargs):
                self._root_index, self._root_index_total = None, -1      # see the module docstring
                return super().initialize_subgame(*args, **kwargs)
        ev.__class__ = FreshRootIndex
        ev._ensure_fused_attrs()

    def store(prefix, batch):
        out[f"{prefix}/len"] = np.int64(len(batch))
        f = batch.features
        out[f"{prefix}/context"] = f.context.numpy()
        out[f"{prefix}/board"] = f.board.numpy()
        out[f"{prefix}/to_act"] = f.to_act.numpy()
        out[f"{prefix}/street"] = f.street.numpy()
        fb = f.beliefs.numpy().reshape(-1, 2, NUM_HANDS)
        out[f"{prefix}/beliefs"] = np.ascontiguousarray(fb[..., cols])
        out[f"{prefix}/beliefs_rowsum"] = fb.astype(np.float64).sum(-1)
        out[f"{prefix}/legal_masks"] = batch.legal_masks.numpy()
        if batch.value_targets is not None:
            vt = batch.value_targets.numpy()
            out[f"{prefix}/value_targets"] = np.ascontiguousarray(vt[..., cols]).astype(np.float32)
            out[f"{prefix}/value_targets_rowsum"] = vt.astype(np.float64).sum(-1)
        if batch.policy_targets is not None:
            pt = batch.policy_targets.numpy()
            out[f"{prefix}/policy_targets"] = np.ascontiguousarray(pt[:, cols, :]).astype(np.float32)
            out[f"{prefix}/policy_targets_sum"] = pt.astype(np.float64).sum(axis=1)

    class Recorder:
        def __init__(self, tag):
            self.tag, self.count = tag, 0

        def add_batch(self, batch):
            store(f"{self.tag}/{self.count}", batch)
            self.count += 1

    value_buffer, policy_buffer = Recorder("value_buffer"), Recorder("policy_buffer")
    dg = RebelDataGenerator(env_proto, ev, value_buffer, policy_buffer)
    for f in ENV_FIELDS:
        out[f"first_deal/{f}"] = getattr(dg.current_pbs.env, f).clone().numpy()
    value_batch, policy_batch = dg.generate_data(ASKED)
    store("returned/value", value_batch)
    store("returned/policy", policy_batch)
    out["last_extra"] = np.int64(dg.last_extra)
    out["passes"] = np.int64(policy_buffer.count)
    for f in ENV_FIELDS:
        out[f"left/{f}"] = getattr(dg.current_pbs.env, f).clone().numpy()
    lb = dg.current_pbs.beliefs.numpy()
    out["left/beliefs"] = np.ascontiguousarray(lb[..., cols]).astype(np.float32)
    out["left/beliefs_rowsum"] = lb.astype(np.float64).sum(-1)
    print("passes", policy_buffer.count, "value adds", value_buffer.count, "returned", len(value_batch), len(policy_batch),
          "last_extra", dg.last_extra, "left", lb.shape[0], "streets", dg.current_pbs.env.street.tolist())
    path = os.path.join(HERE, "fused_generator_golden.npz" if fused else "generator_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path) // 1024, "KiB")


if __name__ == "__main__":
    main(fused="--fused" in sys.argv[1:])
