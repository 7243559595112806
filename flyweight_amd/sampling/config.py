"""Sampling settings of a request, with the reference's names, meanings and validation
(src/flyweight/sampling.py:10-47). The built-in defaults are the reference's command-line
ones: temperature 0.8, top_k 40, top_p 0.95, min_p 0.05; a task submitted to the engine
without settings is greedy with top_k 20, top_p 0.95, min_p 0, as the reference's native
task defaults are (native/src/v2_runtime.cpp:32601-32605). Penalties are not offered."""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

@dataclass(frozen=True)
class SamplingConfig:
    temperature: float = 0.8     # 0 is greedy: the best candidate, ties to the lowest id
    top_k: int = 40              # how many candidates the sampler considers; 0 = all
    top_p: float = 0.95          # nucleus cut over those candidates, in (0, 1]
    min_p: float = 0.05          # drop candidates below this fraction of the best one's probability
    seed: Optional[int] = None   # fixed RNG seed for a sample that reproduces

    def __post_init__(self) -> None:
        if not (self.temperature >= 0 and math.isfinite(self.temperature)):
            raise ValueError("temperature must be non-negative")
        if self.top_k < 0:
            raise ValueError("top_k must be non-negative")
        if not 0 < self.top_p <= 1:
            raise ValueError("top_p must be in (0, 1]")
        if not 0 <= self.min_p <= 1:
            raise ValueError("min_p must be in [0, 1]")

    @property
    def greedy(self) -> bool:
        return not self.temperature > 0


GREEDY = SamplingConfig(temperature=0.0, top_k=20, top_p=0.95, min_p=0.0)


def defaults() -> dict:
    config = SamplingConfig()
    return {"temperature": config.temperature, "top_k": config.top_k, "top_p": config.top_p, "min_p": config.min_p}
