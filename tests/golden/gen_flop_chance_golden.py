"""Writes tests/golden/flop_chance_golden.npz by RUNNING the reference's own
``ChanceNodeHelper`` (src/p2/search/chance_node_helper.py:76-357) and suit maps
(src/p2/env/card_utils.py:153-193) on the CPU of the build container.  Run once, here only:
    python tests/golden/gen_flop_chance_golden.py

Holds the canonical-flop cache (class cards, class sizes, flop -> class), the hand-index suit
permutations, and ``flop_chance_values`` for two deterministic networks — one echoes the
post-chance ranges, one depends on the board's suits and on the hand index, so that a wrong
permutation direction or a wrong canonical representative shows — in three modes: all classes
and all 24 permutations; all classes with 6 drawn permutations per chunk; 256 drawn classes with
6 drawn permutations.  The draws come from a seeded CPU generator; the drawn indices are stored
beside the results (replayed from the same seed) for checkers that do not draw themselves.
"""
from __future__ import annotations

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from gen_cfr_golden import REF_SRC, install_stand_ins  # noqa: E402

SEED = 20240611


def main() -> None:
    os.environ.setdefault("TORCHDYNAMO_DISABLE", "1")
    install_stand_ins()
    sys.path.insert(0, REF_SRC)
    import warnings
    import torch
    from p2.env.card_utils import NUM_HANDS
    from p2.models.mlp.mlp_features import MLPFeatures
    from p2.models.model_output import ModelOutput
    from p2.search.chance_node_helper import ChanceNodeHelper
    warnings.filterwarnings("ignore")

    def output(hv):
        return ModelOutput(policy_logits=torch.zeros(hv.shape[0], 3), value=torch.zeros(hv.shape[0]), hand_values=hv)

    class Echo:
        def eval(self):
            pass

        def __call__(self, f):
            return output(f.beliefs.view(-1, 2, NUM_HANDS).float())

    class SuitAware:
        """range entry x (1 + suit of the first board card / 10 + rank of the third / 100)
        + 0.001 x (hand index mod 7) x (player + 1)"""

        def eval(self):
            pass

        def __call__(self, f):
            b = f.beliefs.view(-1, 2, NUM_HANDS).float()
            w = 1.0 + (f.board[:, 0] // 13).float() / 10.0 + (f.board[:, 2] % 13).float() / 100.0
            h = (torch.arange(NUM_HANDS) % 7).float() * 0.001
            return output(b * w[:, None, None] + h[None, None, :] * torch.tensor([1.0, 2.0])[None, :, None])

    rng = np.random.default_rng(4242)
    n = 3
    pre = rng.gamma(0.5, size=(n, 2, NUM_HANDS)).astype(np.float32)
    pre /= pre.sum(-1, keepdims=True)
    pre[2, 1] = 0.0
    pre[2, 1, 0] = 1.0                                 # a delta range: dead on the flops that block it
    roots = np.array([2, 0], dtype=np.int64)
    feats = MLPFeatures(context=torch.zeros(n, 1), street=torch.zeros(n, dtype=torch.long),
                        to_act=torch.zeros(n, dtype=torch.long), board=torch.full((n, 5), -1, dtype=torch.long),
                        beliefs=torch.zeros(n, 2 * NUM_HANDS))
    out = {"pre_beliefs": pre, "root_indices": roots, "seed": np.int64(SEED)}
    modes = {"all": (0, 0), "all_perm6": (0, 6), "sample256_perm6": (256, 6)}
    for name, model in (("echo", Echo()), ("suit_aware", SuitAware())):
        for mode, (sample, nperm) in modes.items():
            gen = torch.Generator(device="cpu")
            gen.manual_seed(SEED)
            helper = ChanceNodeHelper(device=torch.device("cpu"), float_dtype=torch.float32, num_players=2,
                                      model=model, generator=gen)
            helper.FLOP_SAMPLE_SIZE = sample
            helper.NUM_PERM_SAMPLES = nperm
            got = helper.flop_chance_values(torch.from_numpy(roots), feats, torch.from_numpy(pre.copy()))
            out[f"{name}_{mode}"] = got.numpy().astype(np.float32)
            print(name, mode, got.shape, float(got.abs().sum()))
    # the cache and the suit maps
    out["flop_id_to_canonical"] = helper.flop_id_to_canonical.numpy().astype(np.int8)
    out["flop_id_to_count"] = helper.flop_id_to_count.numpy().astype(np.int16)
    out["flop_to_canon"] = helper.flop_to_canon.numpy().astype(np.int16)
    out["suit_permutations"] = helper.suit_permutations.numpy().astype(np.int8)
    out["combo_perm"] = helper.combo_perm.numpy().astype(np.int16)
    out["combo_perm_inverse"] = helper.combo_perm_inverse.numpy().astype(np.int16)
    out["board_to_flop_id_sample"] = helper.board_to_flop_id[3, 17, 40:52].numpy().astype(np.int16)
    # the draws of each mode, replayed from the seed in the order the helper makes them
    probs = helper.flop_id_to_count.to(torch.float32)
    gen = torch.Generator(device="cpu")
    gen.manual_seed(SEED)
    n_chunks = (helper.flop_id_to_canonical.shape[0] + helper.FLOP_CHUNK_SIZE - 1) // helper.FLOP_CHUNK_SIZE
    out["all_perm6_rows"] = np.stack([torch.randperm(24, generator=gen)[:6].numpy() for _ in range(n_chunks)])
    gen.manual_seed(SEED)
    out["sample256_idx"] = torch.multinomial(probs, 256, replacement=True, generator=gen).numpy().astype(np.int16)
    out["sample256_rows"] = torch.randperm(24, generator=gen)[:6].numpy()[None]
    path = os.path.join(HERE, "flop_chance_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path) // 1024, "KiB")


if __name__ == "__main__":
    main()
