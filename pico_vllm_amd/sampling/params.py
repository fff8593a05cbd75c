"""Per-request sampling options.

``max_new_tokens``, ``temperature`` and ``top_p`` are the arguments of the
reference's ``Engine.submit`` (pico_vllm/engine.py:243-247) with the same
meanings: temperature 0 is greedy, top_p >= 1 switches nucleus filtering off
(sampler.py:92-108).  ``seed`` and ``ignore_eos`` have no counterpart there.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional


@dataclass
class SamplingParams:
    max_new_tokens: int = 16
    temperature: float = 0.0
    top_p: float = 1.0
    seed: Optional[int] = None          # None: derived from the engine's seed and the request id
    ignore_eos: bool = False

    def validate(self) -> None:
        if self.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be at least 1")
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
        if not (0 < self.top_p):
            raise ValueError("top_p must be positive")
