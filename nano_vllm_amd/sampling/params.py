"""Per-request sampling options: the reference's three (nanovllm/sampling_params.py:4-11),
with temperature 0 meaning greedy (the reference forbids it) and an optional seed."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class SamplingParams:
    temperature: float = 1.0
    max_tokens: int = 64
    ignore_eos: bool = False
    seed: Optional[int] = None          # None: the engine's seed

    def __post_init__(self):
        if self.temperature < 0:
            raise ValueError("temperature must be 0 (greedy) or positive")
        if 0 < self.temperature <= 1e-10:
            self.temperature = 0.0       # the reference's lower bound: treat as greedy
        if self.max_tokens <= 0:
            raise ValueError("max_tokens must be positive")
