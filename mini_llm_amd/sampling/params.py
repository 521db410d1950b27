"""How a request samples. The reference's completion script has a temperature and a top-p,
temperature <= 0 meaning greedy (scripts/complete.py:50-52,116-123); the engine itself takes
the argmax (engine/src/argmax.cu)."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0   # 0 (or less): greedy
    top_p: float = 1.0         # nucleus mass; 1: the whole distribution
    seed: int = 0              # the draws are a function of (seed, number of tokens generated so far)

    def __post_init__(self):
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError(f"top_p must be in (0, 1], not {self.top_p}")

    @property
    def greedy(self) -> bool:
        return not self.temperature > 0.0
