"""Flat ReBeL features of public states, MI355X path.

Mirror of ``RebelFeatureEncoder`` (src/p2/models/mlp/rebel_feature_encoder.py:17-127): same
constructor, ``encode(beliefs, pre_chance_node, indices)`` and result.  ``env`` is any object
with the reference env's attribute names as device tensors (``to_act, button, starting_stacks, pot,
committed, actions_this_round, board_indices, last_board_indices``); the evaluator's ``env`` is one.
The context features and the board choice are one HIP kernel (``p2hip_encode_context``); the
beliefs are handed on as a view.
"""
from __future__ import annotations

import torch

from . import _lib
from .card_utils import NUM_HANDS
from .chance_node_helper import MLPFeatures
from ._guards import require as _req


class RebelFeatureEncoder:
    feature_dim: int = 2661
    belief_dim: int = 1326

    def __init__(self, env, device: torch.device | None = None, dtype: torch.dtype | None = None) -> None:
        self.env = env
        self.device = torch.device(device) if device is not None else torch.device(env.to_act.device)
        self.dtype = dtype or torch.float32
        if self.dtype != torch.float32:
            raise ValueError("RebelFeatureEncoder computes float32 features")

    def encode(self, beliefs: torch.Tensor, pre_chance_node: torch.Tensor | bool | None = None,
               indices: torch.Tensor | None = None) -> MLPFeatures:
        """beliefs [B,2,1326] -> MLPFeatures(context [B,4], street zeros [B], to_act [B],
        board [B,5] (the board before the last deal where ``pre_chance_node``), beliefs [B,2652])."""
        dev = self.device
        if indices is not None:
            indices = indices.to(dev)
            beliefs = beliefs[indices]
            if isinstance(pre_chance_node, torch.Tensor):
                pre_chance_node = pre_chance_node[indices]
        return self.encode_rows(beliefs, indices, pre_chance_node)

    def encode_rows(self, beliefs: torch.Tensor, rows: torch.Tensor | None,
                    pre_chance_node: torch.Tensor | bool | None = None) -> MLPFeatures:
        """``encode`` for beliefs (and a mask) that are already those of env rows ``rows``
        (None: all rows, in order)."""
        dev = self.device
        indices = rows.to(dev) if rows is not None else None
        m = beliefs.shape[0]
        if not _lib.hip_is_available():
            raise RuntimeError("RebelFeatureEncoder.encode needs libp2hip.so and a GPU (no CPU fallback exists).")
        _lib.require_gpu(beliefs, "RebelFeatureEncoder.encode")

        widths = {"starting_stacks": 2, "committed": 2, "last_board_indices": 5, "board_indices": 5}

        def get(name: str) -> torch.Tensor:
            val = getattr(self.env, name)
            val = val[indices] if indices is not None else val
            want = (m, widths[name]) if name in widths else (m,)
            if tuple(val.shape) != want:
                raise ValueError(f"env.{name} has shape {tuple(val.shape)}, expected {want}")
            return val.to(device=dev, dtype=torch.int64).contiguous()

        pre_ptr, pre_all, pre_keep = None, 0, None
        if isinstance(pre_chance_node, torch.Tensor):
            pre_keep = pre_chance_node.to(device=dev, dtype=torch.uint8).contiguous()
            _req(pre_keep.shape == (m,), "pre_keep.shape == (m,)")
            pre_ptr = _lib.ptr(pre_keep)
        elif pre_chance_node is not None:
            pre_all = int(bool(pre_chance_node))
        to_act = get("to_act")
        context = torch.empty(m, 4, dtype=torch.float32, device=dev)
        board = torch.empty(m, 5, dtype=torch.int64, device=dev)
        args = [get(n) for n in ("button", "starting_stacks", "pot", "committed", "actions_this_round")]
        last_board, cur_board = get("last_board_indices"), get("board_indices")
        _lib.call("p2hip_encode_context", _lib.ptr(to_act), *[_lib.ptr(a) for a in args], pre_ptr, pre_all,
                  _lib.ptr(last_board), _lib.ptr(cur_board), m, _lib.ptr(context), _lib.ptr(board), _lib.stream_ptr())
        return MLPFeatures(context=context, street=torch.zeros(m, device=dev, dtype=self.dtype), to_act=to_act,
                           board=board, beliefs=beliefs.reshape(-1, 2 * NUM_HANDS))
