"""Search configuration with the reference's field names and defaults
(``SearchConfig`` / ``CFRType`` / ``WarmStartType`` of
src/p2/core/structured_config.py:46-56, :238-265).  Any object exposing the same
attribute names (the reference's hydra ``Config`` included) can be passed to the
evaluator instead."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

from .fused_cfr_hip import CFRType


@dataclass
class SearchConfig:
    enabled: bool = True
    depth: int = 2
    iterations: int = 100
    warm_start_iterations: int = 15
    warm_start_type: str = "model_br"     # model | model_br (structured_config.py:53-55)
    warm_start_multiplier: float = 1.0
    dcfr_alpha: float = 1.5
    dcfr_beta: float = 0.0
    dcfr_gamma: float = 2.0
    dcfr_alpha_final: Optional[float] = None
    dcfr_beta_final: Optional[float] = None
    dcfr_gamma_final: Optional[float] = None
    dcfr_plus_delay: int = 50
    cfr_type: CFRType = CFRType.linear
    cfr_plus: bool = True
    cfr_avg: bool = True
    sample_epsilon: float = 0.25
    value_targets_from_final_policy: bool = False
    sparse: bool = True
    sparse_fused: bool = True


@dataclass
class EnvConfig:
    bet_bins: List[float] = field(default_factory=lambda: [0.5, 1.0])
    bb: int = 100


@dataclass
class ModelConfig:
    num_supervisions: int = 1


@dataclass
class Config:
    num_envs: int = 1
    seed: int = 42
    search: SearchConfig = field(default_factory=SearchConfig)
    env: EnvConfig = field(default_factory=EnvConfig)
    model: ModelConfig = field(default_factory=ModelConfig)


def river_dcfr_config(num_envs: int, iterations: int = 200, depth: int = 2, dcfr_delay: int = 0) -> Config:
    """The synthetic river workload: discounted CFR (alpha 1.5, beta 0, gamma 2), no CFR+,
    no warm start, bins {0.5, 1.0}."""
    return Config(num_envs=num_envs, search=SearchConfig(
        depth=depth, iterations=iterations, warm_start_iterations=0, dcfr_alpha=1.5, dcfr_beta=0.0,
        dcfr_gamma=2.0, dcfr_plus_delay=dcfr_delay, cfr_type=CFRType.discounted, cfr_plus=False, cfr_avg=False))
