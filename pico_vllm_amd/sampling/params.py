"""Per-request sampling options.

``max_new_tokens``, ``temperature`` and ``top_p`` are the arguments of the
reference's ``Engine.submit`` (pico_vllm/engine.py:243-247) with the same
meanings: temperature 0 is greedy, top_p >= 1 switches nucleus filtering off
(sampler.py:92-108).  ``seed``, ``ignore_eos`` and ``stop_token_ids`` (further tokens that end the
request like the end-of-sequence token; the token is kept) have no counterpart there.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from numbers import Integral
from typing import List, Optional


def _whole(x) -> bool:
    return isinstance(x, Integral) and not isinstance(x, bool)


@dataclass
class SamplingParams:
    max_new_tokens: int = 16
    temperature: float = 0.0
    top_p: float = 1.0
    seed: Optional[int] = None          # None: derived from the engine's seed and the request id
    ignore_eos: bool = False
    stop_token_ids: List[int] = field(default_factory=list)

    def validate(self) -> None:
        if not _whole(self.max_new_tokens) or self.max_new_tokens < 1:
            raise ValueError(f"max_new_tokens must be an integer of at least 1, got {self.max_new_tokens!r}")
        if not (0 <= self.temperature < float("inf")):               # refuses not-a-number too
            raise ValueError(f"temperature must be a number that is not negative, got {self.temperature!r}")
        if not (0 < self.top_p < float("inf")):
            raise ValueError(f"top_p must be a positive number, got {self.top_p!r}")
        if not all(_whole(t) for t in self.stop_token_ids):
            raise ValueError(f"stop_token_ids must be token ids, got {self.stop_token_ids!r}")
