"""The scheduler: which requests run in the next step and with how many tokens.

First come, first served, as in the reference (pico_vllm/scheduler.py:174-178:
``waiting.pop(0)`` while fewer than ``max_num_seqs`` are in progress).  What
the reference does not have: a token budget per step with prompts cut into
portions of at most ``prefill_chunk`` tokens (it prefills whole prompts, engine.py:305-306), admission that looks
at free pages (its ``can_allocate_gpu`` is unused, blockmanager.py:173-176),
and a decision for the moment pages run out (there the allocation raises from
inside the step, blockmanager.py:77-78).

When pages run out: the running request that was admitted last is preempted:
its pages and state slot are given back, it returns to the FRONT of the
waiting queue keeping the tokens it has generated, and on readmission it runs
prompt + generated tokens again as one prompt (recomputation).  A request that
could not fit even alone in an empty pool is refused when it is added.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Deque, List, Optional

from ..cache.manager import CacheManager
from .request import Request, RequestStatus


@dataclass
class ScheduledSeq:
    request: Request
    num_tokens: int          # tokens all_ids[num_computed : num_computed + num_tokens] run in this step

    @property
    def samples(self) -> bool:
        """The step includes the request's last token, so its logits give the next token."""
        return self.request.num_computed + self.num_tokens == self.request.total_len


@dataclass
class SchedulerOutput:
    seqs: List[ScheduledSeq] = field(default_factory=list)
    preempted: List[Request] = field(default_factory=list)

    @property
    def num_tokens(self) -> int:
        return sum(s.num_tokens for s in self.seqs)


class Scheduler:
    def __init__(self, manager: CacheManager, max_num_seqs: int = 4, max_num_batched_tokens: int = 2048,
                 max_seq_len: int = 4096, prefill_chunk: Optional[int] = None):
        if max_num_batched_tokens < max_num_seqs:
            raise ValueError("max_num_batched_tokens must be at least max_num_seqs, or decoding requests starve")
        if prefill_chunk is not None and prefill_chunk < 1:
            raise ValueError("prefill_chunk must be positive")
        self.manager = manager
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens
        # the longest portion of one prompt in a step (beside the budget, which all sequences of a step share)
        self.prefill_chunk = min(prefill_chunk or max_num_batched_tokens, max_num_batched_tokens)
        self.max_seq_len = max_seq_len
        self.waiting: Deque[Request] = deque()
        self.running: List[Request] = []          # in order of admission
        self.num_preemptions = 0

    # ---- queue ----------------------------------------------------------
    def add_request(self, req: Request) -> None:
        longest = len(req.input_ids) + req.params.max_new_tokens
        if not req.input_ids:
            raise ValueError("a request needs at least one prompt token")
        if longest > self.max_seq_len:
            raise ValueError(f"request {req.request_id}: prompt + max_new_tokens = {longest} exceeds "
                             f"max_seq_len = {self.max_seq_len}")
        P = self.manager.page_size
        for g in self.manager.groups:
            pages = -(-longest // P)
            if g.window > 0:
                # a group with a window holds the window and the step's own tokens, whatever the length: pages that
                # the window has passed went back before the step
                pages = min(pages, -(-(g.window + self.prefill_chunk) // P) + 1)
            if pages > g.pool.num_pages:
                raise ValueError(f"request {req.request_id} needs {pages} pages at its longest; the pool has "
                                 f"{g.pool.num_pages}, so it could never finish")
        req.status = RequestStatus.WAITING
        self.waiting.append(req)

    def has_unfinished(self) -> bool:
        return bool(self.waiting or self.running)

    # ---- one decision ---------------------------------------------------
    def schedule(self) -> SchedulerOutput:
        out = SchedulerOutput()
        budget = self.max_num_batched_tokens
        # 1. requests already running: decoding ones first, then those still in their prompt
        order = sorted(self.running, key=lambda r: (r.num_uncomputed != 1,))
        for req in order:
            if req.status is not RequestStatus.RUNNING or budget <= 0:
                continue
            n = min(req.num_uncomputed, budget, self.prefill_chunk)
            while not self.manager.grow(req.request_id, req.num_computed + n):
                victim = self.running[-1]
                self._preempt(victim, out)
                if victim is req:
                    break
            if req.status is not RequestStatus.RUNNING:
                continue
            out.seqs.append(ScheduledSeq(req, n))
            budget -= n
        # a request scheduled above may have been preempted later to make room for an older one
        out.seqs = [s for s in out.seqs if s.request.status is RequestStatus.RUNNING]
        # 2. admit waiting requests in order while everything they need is there
        while self.waiting and len(self.running) < self.max_num_seqs and budget > 0 and not out.preempted:
            req = self.waiting[0]
            n = min(req.num_uncomputed, budget, self.prefill_chunk)
            if not self.manager.add_request(req.request_id):
                break
            if not self.manager.grow(req.request_id, n):
                self.manager.free_request(req.request_id)
                break
            self.waiting.popleft()
            req.status = RequestStatus.RUNNING
            self.running.append(req)
            out.seqs.append(ScheduledSeq(req, n))
            budget -= n
        return out

    def _preempt(self, victim: Request, out: SchedulerOutput) -> None:
        self.manager.free_request(victim.request_id)
        self.running.remove(victim)
        victim.status = RequestStatus.WAITING
        victim.num_computed = 0
        victim.num_preemptions += 1
        self.num_preemptions += 1
        self.waiting.appendleft(victim)
        out.preempted.append(victim)

    # ---- after a step ---------------------------------------------------
    def on_step_done(self, seq: ScheduledSeq) -> None:
        req = seq.request
        req.num_computed += seq.num_tokens
        self.manager.advance(req.request_id, req.num_computed)

    def finish(self, req: Request, reason: str) -> None:
        """The request is done: its pages and state slot go back in this same step
        (the reference releases one step later, pico_vllm/engine.py:426-428)."""
        if req in self.running:
            self.manager.free_request(req.request_id)
            self.running.remove(req)
        else:                      # preempted while its last token was still on the device: it holds nothing
            self.waiting.remove(req)
        req.status = RequestStatus.FINISHED
        req.finish_reason = reason
