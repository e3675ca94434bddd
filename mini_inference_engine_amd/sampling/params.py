"""Per-request sampling options, as the reference names them
(inference_engine/sampling.py:6-10), plus a seed."""
from __future__ import annotations

from dataclasses import dataclass


@dataclass
class SamplingParams:
    max_tokens: int = 128
    temperature: float = 0.0        # 0 = greedy
    ignore_eos: bool = False        # keep generating past the stop token
    seed: int | None = None         # noise stream of this request; None: derived from the engine's seed

    def __post_init__(self):
        if self.max_tokens < 0:
            raise ValueError("max_tokens must be >= 0")
        if self.temperature < 0:
            raise ValueError("temperature must be >= 0")
