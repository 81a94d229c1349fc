"""Container of training samples handed from the search to the replay buffers.

Mirror of ``RebelBatch`` (src/p2/rl/rebel_batch.py:16-70 and its ``cat``): features, legal
masks, policy and / or value targets, per-sample statistics; indexing, device moves and
concatenation.  The suit-permutation augmentation of the trainer is not part of this package.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import torch

from .chance_node_helper import MLPFeatures
from ._guards import require as _req


@dataclass
class RebelBatch:
    features: MLPFeatures
    legal_masks: torch.Tensor
    policy_targets: Optional[torch.Tensor] = None
    value_targets: Optional[torch.Tensor] = None
    statistics: dict[str, torch.Tensor] = field(default_factory=dict)

    def __post_init__(self) -> None:
        _req(self.value_targets is not None or self.policy_targets is not None,
             "self.value_targets is not None or self.policy_targets is not None")
        n = len(self.features)
        _req(n == self.legal_masks.shape[0], "n == self.legal_masks.shape[0]")
        if self.policy_targets is not None:
            _req(n == self.policy_targets.shape[0], "n == self.policy_targets.shape[0]")
        if self.value_targets is not None:
            _req(n == self.value_targets.shape[0], "n == self.value_targets.shape[0]")
        for key in self.statistics:
            _req(n == self.statistics[key].shape[0], key)

    def __len__(self) -> int:
        return len(self.features)

    def __getitem__(self, idx) -> "RebelBatch":
        return RebelBatch(
            features=self.features[idx],
            policy_targets=self.policy_targets[idx] if self.policy_targets is not None else None,
            value_targets=self.value_targets[idx] if self.value_targets is not None else None,
            legal_masks=self.legal_masks[idx],
            statistics={k: v[idx] for k, v in self.statistics.items()})

    def to(self, device) -> "RebelBatch":
        return RebelBatch(
            features=self.features.to(device),
            policy_targets=self.policy_targets.to(device) if self.policy_targets is not None else None,
            value_targets=self.value_targets.to(device) if self.value_targets is not None else None,
            legal_masks=self.legal_masks.to(device),
            statistics={k: v.to(device) for k, v in self.statistics.items()})

    @classmethod
    def cat(cls, batches: list["RebelBatch"]) -> "RebelBatch":
        """Concatenation; targets must be all present or all absent, statistics follow the keys
        of the first batch (rebel_batch.py:127-167)."""
        if not batches:
            raise ValueError("Cannot concatenate an empty list of batches.")
        if any(b is None for b in batches):
            raise ValueError("Cannot concatenate a list of batches with None values.")
        policy_targets = None
        if batches[0].policy_targets is not None:
            if any(b.policy_targets is None for b in batches):
                raise ValueError("Policy targets must be all present or all absent.")
            policy_targets = torch.cat([b.policy_targets for b in batches], dim=0)
        value_targets = None
        if batches[0].value_targets is not None:
            if any(b.value_targets is None for b in batches):
                raise ValueError("Value targets must be all present or all absent.")
            value_targets = torch.cat([b.value_targets for b in batches], dim=0)
        return cls(
            features=MLPFeatures.cat([b.features for b in batches]),
            legal_masks=torch.cat([b.legal_masks for b in batches], dim=0),
            policy_targets=policy_targets, value_targets=value_targets,
            statistics={k: torch.cat([b.statistics[k] for b in batches], dim=0) for k in batches[0].statistics})
