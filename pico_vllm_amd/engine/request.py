"""A generation request and its state.

States in the reference: WAITING / PREFILL / DECODING / FINISHED / CLOSED
(pico_vllm/scheduler.py:7-12).  Here a running request is prefilling while
``num_computed < len(all tokens) - 0`` still leaves prompt tokens to run, and
there is no separate CLOSED: a request gives its pages back in the step in
which it finishes.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum
from typing import List, Optional

from ..sampling.params import SamplingParams


class RequestStatus(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


@dataclass
class Request:
    request_id: int
    input_ids: List[int]
    params: SamplingParams
    seed: int = 0
    generated_ids: List[int] = field(default_factory=list)
    status: RequestStatus = RequestStatus.WAITING
    finish_reason: Optional[str] = None       # "eos" or "length"
    num_computed: int = 0                     # tokens whose keys are in the cache
    num_preemptions: int = 0
    num_pending: int = 0                      # tokens sampled on the device whose values the host has not read yet (up to 2)

    @property
    def all_ids(self) -> List[int]:
        return self.input_ids + self.generated_ids

    @property
    def total_len(self) -> int:
        return len(self.input_ids) + len(self.generated_ids) + self.num_pending

    @property
    def num_generated(self) -> int:
        return len(self.generated_ids) + self.num_pending

    @property
    def num_uncomputed(self) -> int:
        """Tokens not yet in the cache; the last of them yields the next sample."""
        return self.total_len - self.num_computed

    def is_max_len_finished(self) -> bool:
        # the first sampled token counts (pico_vllm/scheduler.py:55-56)
        return self.num_generated >= self.params.max_new_tokens
