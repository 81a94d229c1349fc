"""Writes tests/golden/chance_golden.npz by RUNNING the reference's own
``ChanceNodeHelper.single_card_chance_values`` (src/p2/search/chance_node_helper.py:360-479) on
the CPU of the build container.  Run once, here only:  python tests/golden/gen_chance_golden.py

The reference's tests for this method check shapes only, so these vectors are what pins the
masking / renormalisation / sample order / mean against the reference.  Two deterministic
networks in the style of its tests (tests/test_chance_node_helper.py:46-117): one echoes the
post-chance ranges, one returns a function of the sample's board.  hydra / omegaconf (imported by
``p2.core.structured_config`` to register a dataclass) are replaced by empty stand-in modules.
"""
from __future__ import annotations

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from gen_cfr_golden import REF_SRC, install_stand_ins  # noqa: E402


def main() -> None:
    os.environ.setdefault("TORCHDYNAMO_DISABLE", "1")
    install_stand_ins()
    sys.path.insert(0, REF_SRC)
    import torch
    from p2.env.card_utils import NUM_HANDS
    from p2.models.mlp.mlp_features import MLPFeatures
    from p2.models.model_output import ModelOutput
    from p2.search.chance_node_helper import ChanceNodeHelper

    class Echo:
        def eval(self):
            pass

        def __call__(self, f):
            b = f.beliefs.view(-1, 2, NUM_HANDS).float()
            return ModelOutput(policy_logits=torch.zeros(b.shape[0], 3), value=torch.zeros(b.shape[0]), hand_values=b)

    class BoardAndRange:
        """hand value = range entry x (1 + rank sum of the board / 100): depends on both inputs."""

        def eval(self):
            pass

        def __call__(self, f):
            b = f.beliefs.view(-1, 2, NUM_HANDS).float()
            ranks = torch.where(f.board >= 0, (f.board % 13).float(), torch.zeros_like(f.board, dtype=torch.float32))
            w = 1.0 + ranks.sum(dim=1) / 100.0
            return ModelOutput(policy_logits=torch.zeros(b.shape[0], 3), value=torch.zeros(b.shape[0]),
                               hand_values=b * w[:, None, None])

    rng = np.random.default_rng(77)
    n = 6
    board = np.full((n, 5), -1, dtype=np.int64)
    for i, k in enumerate([4, 4, 3, 4, 3, 4]):
        board[i, :k] = rng.permutation(52)[:k]
    pre = rng.gamma(0.5, size=(n, 2, NUM_HANDS)).astype(np.float32)
    pre /= pre.sum(-1, keepdims=True)
    pre[1, 0] = 0.0                                   # a dead range: uniform fallback on every sample
    pre[3, 1] = 0.0
    pre[3, 1, 200] = 1.0                              # a delta range: dead only where a sample blocks it
    roots = np.array([5, 0, 3, 1, 2], dtype=np.int64)
    feats = MLPFeatures(context=torch.zeros(n, 1), street=torch.full((n,), 3, dtype=torch.long),
                        to_act=torch.zeros(n, dtype=torch.long), board=torch.from_numpy(board.copy()),
                        beliefs=torch.zeros(n, 2 * NUM_HANDS))
    out = {"board": board, "pre_beliefs": pre, "root_indices": roots}
    for name, model in (("echo", Echo()), ("board_and_range", BoardAndRange())):
        helper = ChanceNodeHelper(device=torch.device("cpu"), float_dtype=torch.float32, num_players=2, model=model)
        got = helper.single_card_chance_values(torch.from_numpy(roots), feats, torch.from_numpy(pre.copy()),
                                               torch.from_numpy(board.copy()))
        out[name] = got.numpy().astype(np.float32)
        print(name, got.shape, float(got.abs().sum()))
    path = os.path.join(HERE, "chance_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path) // 1024, "KiB")


if __name__ == "__main__":
    main()
