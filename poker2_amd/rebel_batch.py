"""Container of training samples handed from the search to the replay buffers.

Same fields and behaviour as ``RebelBatch`` (src/p2/rl/rebel_batch.py:16-70 and its ``cat``,
:127-167): features, legal masks, policy and / or value targets, per-sample statistics; indexing,
device moves and concatenation.  Every operation is one map over the batch's per-sample parts
(``_map``), so a field added to the container needs no further code.  The suit-permutation
augmentation of the trainer is not part of this package.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Optional

import torch

from .chance_node_helper import MLPFeatures
from ._guards import require as _req

_TARGETS = ("policy_targets", "value_targets")


@dataclass
class RebelBatch:
    features: MLPFeatures
    legal_masks: torch.Tensor
    policy_targets: Optional[torch.Tensor] = None
    value_targets: Optional[torch.Tensor] = None
    statistics: dict[str, torch.Tensor] = field(default_factory=dict)

    def __post_init__(self) -> None:
        _req(any(getattr(self, t) is not None for t in _TARGETS), "a batch carries policy targets, value targets or both")
        n = len(self.features)
        rows = {"legal_masks": self.legal_masks, **{t: getattr(self, t) for t in _TARGETS}, **self.statistics}
        for name, part in rows.items():
            _req(part is None or part.shape[0] == n, f"{name}: one row per sample")

    def __len__(self) -> int:
        return len(self.features)

    def _map(self, on_features: Callable, on_tensor: Callable) -> "RebelBatch":
        """A batch whose features went through ``on_features`` and whose tensors through ``on_tensor``."""
        def opt(x):
            return None if x is None else on_tensor(x)
        return RebelBatch(features=on_features(self.features), legal_masks=on_tensor(self.legal_masks),
                          policy_targets=opt(self.policy_targets), value_targets=opt(self.value_targets),
                          statistics={k: on_tensor(v) for k, v in self.statistics.items()})

    def __getitem__(self, idx) -> "RebelBatch":
        return self._map(lambda f: f[idx], lambda x: x[idx])

    def to(self, device) -> "RebelBatch":
        return self._map(lambda f: f.to(device), lambda x: x.to(device))

    @classmethod
    def cat(cls, batches: list["RebelBatch"]) -> "RebelBatch":
        """Concatenation along the sample axis.  A kind of target is carried by all batches or by none;
        the statistics are those the first batch has."""
        if not batches:
            raise ValueError("Cannot concatenate an empty list of batches.")
        if any(b is None for b in batches):
            raise ValueError("Cannot concatenate a list of batches with None values.")
        first = batches[0]

        def joined(pick: Callable) -> torch.Tensor:
            return torch.cat([pick(b) for b in batches], dim=0)
        targets = {}
        for t in _TARGETS:
            have = [getattr(b, t) is not None for b in batches]
            if any(have) != all(have):
                raise ValueError(f"{t.replace('_', ' ').capitalize()} must be all present or all absent.")
            targets[t] = joined(lambda b, t=t: getattr(b, t)) if have[0] else None
        return cls(features=MLPFeatures.cat([b.features for b in batches]), legal_masks=joined(lambda b: b.legal_masks),
                   statistics={k: joined(lambda b, k=k: b.statistics[k]) for k in first.statistics}, **targets)
