"""Per-request sampling options.

``max_new_tokens``, ``temperature`` and ``top_p`` are the arguments of the
reference's ``Engine.submit`` (pico_vllm/engine.py:243-247) with the same
meanings: temperature 0 is greedy, top_p >= 1 switches nucleus filtering off
(sampler.py:92-108).  ``seed``, ``ignore_eos`` and ``stop_token_ids`` (further tokens that end the
request like the end-of-sequence token; the token is kept) have no counterpart there.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional


@dataclass
class SamplingParams:
    max_new_tokens: int = 16
    temperature: float = 0.0
    top_p: float = 1.0
    seed: Optional[int] = None          # None: derived from the engine's seed and the request id
    ignore_eos: bool = False
    stop_token_ids: List[int] = field(default_factory=list)

    def validate(self) -> None:
        if self.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be at least 1")
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
        if not (0 < self.top_p):
            raise ValueError("top_p must be positive")
