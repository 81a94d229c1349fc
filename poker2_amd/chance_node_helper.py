"""Chance-node enumeration around the leaf value network, MI355X path.

Mirror of ``ChanceNodeHelper.single_card_chance_values``
(src/p2/search/chance_node_helper.py:360-479) and of the ``MLPFeatures`` container it hands
to the network (src/p2/models/mlp/mlp_features.py:13-62): same names, arguments, sample
order (state-major, next card ascending) and return value.  The masking / renormalising
expansion and the per-state mean run as HIP kernels (``p2hip_chance_expand``,
``p2hip_chance_mean``); the network itself stays an ordinary PyTorch module.
``flop_chance_values`` (three-card chance nodes through the canonical-flop cache) is not
part of this package.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

from . import _lib
from .card_utils import NUM_HANDS


@dataclass
class MLPFeatures:
    """Feature bundle of the value network (src/p2/models/mlp/mlp_features.py:13-62)."""

    context: torch.Tensor   # [N, C]
    street: torch.Tensor    # [N]
    to_act: torch.Tensor    # [N]
    board: torch.Tensor     # [N, 5] card ids, -1 = not dealt
    beliefs: torch.Tensor   # [N, 2 * 1326]

    def __post_init__(self) -> None:
        n = self.context.shape[0]
        assert self.street.shape == (n,)
        assert self.to_act.shape == (n,)
        assert self.board.shape == (n, 5)
        assert self.beliefs.shape == (n, 2 * NUM_HANDS)

    def __len__(self) -> int:
        return self.context.shape[0]

    def __getitem__(self, index) -> "MLPFeatures":
        return MLPFeatures(context=self.context[index], street=self.street[index], to_act=self.to_act[index],
                           board=self.board[index], beliefs=self.beliefs[index])

    def to(self, device) -> "MLPFeatures":
        return MLPFeatures(context=self.context.to(device), street=self.street.to(device),
                           to_act=self.to_act.to(device), board=self.board.to(device),
                           beliefs=self.beliefs.to(device))

    def clone(self) -> "MLPFeatures":
        return MLPFeatures(context=self.context.clone(), street=self.street.clone(), to_act=self.to_act.clone(),
                           board=self.board.clone(), beliefs=self.beliefs.clone())


def chance_expand(pre_chance_beliefs: torch.Tensor, root_indices: torch.Tensor, board_pre: torch.Tensor,
                  cards_on_board: int | None = None):
    """Every (state, next card) sample of a single-card chance node.

    pre_chance_beliefs [R,2,1326] fp32, board_pre [R,5] int64 (-1 = empty), root_indices [B].
    Returns (post_beliefs [S,2,1326], board_samples [S,5], root_lookup [S], sample_offsets [B+1])
    with samples in (state, card) ascending order.  ``cards_on_board`` (same count for every
    selected state) skips the device-to-host read of the sample count.
    """
    if not _lib.hip_is_available():
        raise RuntimeError("chance_expand needs libp2hip.so and a GPU (no CPU fallback exists).")
    _lib.require_gpu(pre_chance_beliefs, "chance_expand")
    dev = pre_chance_beliefs.device
    assert pre_chance_beliefs.dim() == 3 and tuple(pre_chance_beliefs.shape[1:]) == (2, NUM_HANDS)
    assert board_pre.dim() == 2 and board_pre.shape[1] == 5
    pre = pre_chance_beliefs.contiguous().float()
    board = board_pre.to(device=dev, dtype=torch.int64).contiguous()
    roots = root_indices.to(device=dev, dtype=torch.int64).contiguous()
    b = roots.numel()
    on_board = ((board[roots] >= 0) & (board[roots] < 52)).sum(dim=1)
    offsets = torch.zeros(b + 1, dtype=torch.int64, device=dev)
    torch.cumsum(52 - on_board, dim=0, out=offsets[1:])
    if cards_on_board is None:
        if b and int(on_board.max().item()) >= 5:
            raise ValueError("single-card chance expansion needs an empty board slot (at most 4 cards dealt)")
        total = int(offsets[-1].item()) if b else 0
    else:
        if not 0 <= cards_on_board <= 4:
            raise ValueError("cards_on_board must be in 0..4")
        total = b * (52 - cards_on_board)
    post = torch.empty(total, 2, NUM_HANDS, dtype=torch.float32, device=dev)
    board_samples = torch.empty(total, 5, dtype=torch.int64, device=dev)
    root_lookup = torch.empty(total, dtype=torch.int64, device=dev)
    _lib.call("p2hip_chance_expand", _lib.ptr(pre), _lib.ptr(roots), _lib.ptr(board), b, _lib.ptr(offsets),
              _lib.ptr(post), _lib.ptr(board_samples), _lib.ptr(root_lookup), _lib.stream_ptr())
    return post, board_samples, root_lookup, offsets


def chance_mean(hand_values: torch.Tensor, sample_offsets: torch.Tensor) -> torch.Tensor:
    """[S,2,1326] network outputs -> [B,2,1326] mean over each state's samples."""
    if not _lib.hip_is_available():
        raise RuntimeError("chance_mean needs libp2hip.so and a GPU (no CPU fallback exists).")
    _lib.require_gpu(hand_values, "chance_mean")
    assert hand_values.dim() == 3 and tuple(hand_values.shape[1:]) == (2, NUM_HANDS)
    hv = hand_values.contiguous().float()
    offsets = sample_offsets.to(device=hv.device, dtype=torch.int64).contiguous()
    b = offsets.numel() - 1
    out = torch.empty(b, 2, NUM_HANDS, dtype=torch.float32, device=hv.device)
    _lib.call("p2hip_chance_mean", _lib.ptr(hv), _lib.ptr(offsets), b, _lib.ptr(out), _lib.stream_ptr())
    return out


class ChanceNodeHelper:
    """Utilities for enumerating chance nodes when generating value targets
    (src/p2/search/chance_node_helper.py:31-75; the canonical-flop cache is not built)."""

    def __init__(self, device: torch.device, float_dtype: torch.dtype, num_players: int, model: Any,
                 generator: torch.Generator | None = None, autocast_dtype: torch.dtype | None = torch.float16) -> None:
        if num_players != 2:
            raise ValueError("heads-up only: num_players must be 2")
        self.device = torch.device(device)
        self.float_dtype = float_dtype
        self.num_players = num_players
        self.model = model
        self.generator = generator
        self.autocast_dtype = autocast_dtype   # the reference runs the network under fp16 autocast (:460)

    def flop_chance_values(self, *args, **kwargs):
        raise NotImplementedError("three-card chance nodes (canonical-flop cache) are not part of this package")

    @torch.no_grad()
    def single_card_chance_values(self, root_indices: torch.Tensor, root_features: MLPFeatures,
                                  pre_chance_beliefs: torch.Tensor, board_pre: torch.Tensor,
                                  cards_on_board: int | None = None) -> torch.Tensor:
        """Expected network values over a single-card chance node (turn or river card)."""
        if root_indices.numel() == 0:
            return torch.zeros(0, self.num_players, NUM_HANDS, device=self.device, dtype=self.float_dtype)
        root_indices = root_indices.to(self.device)
        post, board_samples, root_lookup, offsets = chance_expand(pre_chance_beliefs, root_indices, board_pre,
                                                                  cards_on_board)
        if post.shape[0] == 0:
            return torch.zeros(root_indices.numel(), self.num_players, NUM_HANDS, device=self.device,
                               dtype=self.float_dtype)
        src = root_indices[root_lookup]
        synthetic_features = MLPFeatures(
            context=root_features.context[src],
            street=root_features.street[src],
            to_act=root_features.to_act[src],
            board=board_samples,
            beliefs=post.reshape(post.shape[0], -1).to(self.float_dtype),
        )
        model = self.model
        if hasattr(model, "eval"):
            model.eval()
        if self.autocast_dtype is not None:
            with torch.autocast(device_type="cuda", dtype=self.autocast_dtype):
                hand_values = model(synthetic_features).hand_values
        else:
            hand_values = model(synthetic_features).hand_values
        expected = chance_mean(hand_values.to(torch.float32), offsets)
        return expected.to(self.float_dtype)
