"""The step function: run one batch of (request, its next tokens) through the
model from the cache and return the logits at the wanted places.

There is one step for every mixture of prompt portions and single decode
tokens.  The reference has no such function: it prefills each request alone
and whole (pico_vllm/engine.py:299-357) and then decodes all decoding requests
together (:403-410) through two different model entry points.

A pure-decode step whose batch fits ``max_batch_size`` replays a HIP graph
captured for its size (the reference captures one CUDA graph at a fixed batch
of 8, engine.py:98-137).  A step that is one prompt portion alone replays a
graph too, recorded at the next of a few sizes and padded to it with filler
tokens in a sequence of their own: such a step is a few hundred launches and
library calls that cost the host more than they cost the GPU (4.1 ms against
1.6 ms for 300 tokens of the 1.5B shape).  So does a step of a few decoding
requests and one prompt portion of up to ``MIXED_GRAPH_TOKENS`` tokens (what
continuous serving under a small token budget consists of), its single tokens
padded to a power of two as in a decode step.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache.manager import CacheManager
from ..cache.storage import CacheStorage
from ..parts.model import DecoderModel
from .batch import BatchBuffers, BatchError, SeqStep, build_context


def _bucket(n: int) -> int:
    b = 1
    while b < n:
        b *= 2
    return b


def prompt_sizes(most: int) -> List[int]:
    """The sizes at which prompt steps are recorded: 16, 32, 64, then steps of 64 to 512, of 128 to 1,024 and of
    256 beyond, up to ``most``, and ``most`` itself (a step's token budget: the size of most portions of a long
    prompt): less than half of a recorded step is filler for portions of 16 tokens or more, a third from 128 on,
    a fifth from 512 on."""
    out = [16, 32]
    n = 64
    while n <= most:
        out.append(n)
        n += 64 if n < 512 else 128 if n < 1024 else 256
    out = [s for s in out if s <= most]
    if most >= 2 and most not in out:
        out.append(most)
    return out


# A step of single tokens and one prompt portion is recorded only up to this many tokens of the portion: beyond it
# the GPU's work outweighs what the launches cost the host, and every recorded shape costs two warm-up runs.
MIXED_GRAPH_TOKENS = 1024


class ModelRunner:
    def __init__(self, model: DecoderModel, page_size: int, num_pages: int, max_seqs: int,
                 max_tokens_per_step: int, max_seq_len: int, use_graph: bool = False, max_graph_batch: int = 8,
                 graph_prompts: bool = True):
        self.model = model
        self.device = model.device
        specs = model.cache_specs()
        self.manager = CacheManager(specs, page_size, num_pages, max_seqs)
        self.storage = CacheStorage(self.manager, specs, model.dtype, self.device)
        self.max_pages = -(-max_seq_len // page_size)
        self.max_seq_len = max_seq_len
        # a decode batch is padded to the power of two its graph was captured at: rows for that too
        # (and a recorded prompt step has a sequence of filler, and may have padded single tokens in front)
        padded = _bucket(min(max_seqs, max_graph_batch))
        rows = max(max_seqs, padded + 2) if use_graph else max_seqs
        self.buffers = BatchBuffers(self.device, max(max_tokens_per_step + (padded if use_graph else 0), rows), rows,
                                    self.max_pages, max(1, len(self.manager.groups)))
        # a part that decides on the host per step (``Part.graph_safe`` False) keeps the whole model out of graphs
        self.use_graph = use_graph and model.is_graph_safe()
        self.graph_prompts = self.use_graph and graph_prompts and model.is_graph_safe(prompts=True)
        self.prompt_sizes = prompt_sizes(min(max_tokens_per_step, self.max_pages * page_size))
        self.max_graph_batch = max_graph_batch
        self._graphs: Dict[int, tuple] = {}
        # (padded single tokens, recorded size of the portion, its wanted rows, the parts' choices) -> (graph, logits)
        self._prompt_graphs: Dict[tuple, tuple] = {}
        # all graphs take their intermediate tensors from one pool (they never run at the same time), so that a
        # dozen recorded sizes hold the memory of the largest, not of all
        self._graph_pool = torch.cuda.graph_pool_handle() if self.use_graph else None
        self.steps = 0
        self.tokens = 0

    # ---- one step -------------------------------------------------------
    def step(self, seqs: List[SeqStep], device_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Logits float32 [wanted, vocab] in the order of ``seqs`` and their ``want``.

        Pages for the new tokens must have been allocated (``manager.grow``);
        afterwards the caller records the new lengths (``manager.advance``).
        ``device_tokens``: for a step of single tokens, int32 on the device whose entry b is the
        token of sequence b; it replaces the (then meaningless) token ids of ``seqs``, so that
        a decode step can start before the host knows the tokens the step before it sampled."""
        if device_tokens is not None and any(len(s.tokens) != 1 for s in seqs):
            raise BatchError("tokens from the device stand for single-token sequences only")
        for s in seqs:
            if self.manager.num_computed(s.req) + len(s.tokens) > self.max_seq_len:
                raise BatchError(f"request {s.req!r} would grow beyond max_seq_len={self.max_seq_len}")
        # state slots that new requests took start from zero; outside any graph
        self.storage.reset_state(self.manager.take_fresh_slots())
        decode_only = all(len(s.tokens) == 1 and list(s.want) == [0] for s in seqs)
        back = None
        if not decode_only:
            # Single-token sequences first: the attention then serves them through the decode kernel, whoever
            # ordered the batch (the scheduler does so itself; a replayed trace may not).  The logits go back
            # into the caller's order below; what a row holds does not depend on where it stood.
            order = sorted(range(len(seqs)), key=lambda i: len(seqs[i].tokens) != 1)
            if order != list(range(len(seqs))):
                first_row, at = {}, 0
                for i in order:
                    first_row[i] = at
                    at += len(seqs[i].want)
                back = [first_row[i] + j for i in range(len(seqs)) for j in range(len(seqs[i].want))]
                seqs = [seqs[i] for i in order]
        size = self._prompt_size(seqs) if self.graph_prompts and not decode_only else 0
        if self.use_graph and decode_only and len(seqs) <= self.max_graph_batch:
            logits = self._step_graph(seqs, device_tokens)
        elif size:
            logits = self._step_prompt_graph(seqs, size)
            if back is not None:
                logits = logits.index_select(0, torch.tensor(back, dtype=torch.long, device=logits.device))
        else:
            ctx = build_context(seqs, self.manager, self.buffers, self.model.dtype, self.model.spec.vocab_size)
            # the kernel choices of a recorded step for its single tokens (how their contexts are split over
            # workgroups) hold for any context; a step that is not replayed makes the same ones, so that a decoding
            # request gets the same tokens with and without graphs.  (A recorded prompt step equals the same PADDED
            # step unrecorded bit for bit; against the unpadded step that holds only while every product of the
            # step is one of this package's, in which a row does not depend on the rows beside it: up to 64 rows.
            # The library's products may round a row differently at another row count.)
            ctx.max_context = self.max_seq_len
            if device_tokens is not None:
                ctx.token_ids[:len(seqs)].copy_(device_tokens[:len(seqs)])
            logits = self.model.forward(ctx, self.storage)
            if back is not None and logits.shape[0]:
                logits = logits.index_select(0, torch.tensor(back, dtype=torch.long, device=logits.device))
        self.steps += 1
        self.tokens += sum(len(s.tokens) for s in seqs)
        return logits

    def advance(self, seqs: List[SeqStep]) -> None:
        for s in seqs:
            self.manager.advance(s.req, self.manager.num_computed(s.req) + len(s.tokens))

    # ---- graph replay of decode steps -----------------------------------
    def _step_graph(self, seqs: List[SeqStep], device_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        B = len(seqs)
        size = _bucket(B)
        if size not in self._graphs:
            self._capture(size, seqs)
        graph, out = self._graphs[size]
        ctx = build_context(seqs, self.manager, self.buffers, self.model.dtype, self.model.spec.vocab_size, pad_to=size)
        if device_tokens is not None:
            ctx.token_ids[:B].copy_(device_tokens[:B])
        graph.replay()
        return out[:B]

    # ---- graph replay of a prompt portion, alone or behind single tokens --
    def _prompt_size(self, seqs: List[SeqStep]) -> int:
        """The recorded size that serves this step's prompt portion, or 0.  What is recorded: one sequence of two
        tokens or more with at most one wanted row, alone or behind single tokens (each wanted, no more of them than
        a recorded decode step takes) if the portion is short enough for the launches to outweigh the work.  (The
        filler is a sequence of its own with positions from 0, so it needs no room behind the request's tokens.)"""
        last = seqs[-1]
        if len(last.tokens) < 2 or len(last.want) > 1:
            return 0
        singles = len(seqs) - 1
        if singles and (singles > self.max_graph_batch or any(len(s.tokens) != 1 or list(s.want) != [0] for s in seqs[:-1])):
            return 0
        n = len(last.tokens)
        for size in self.prompt_sizes:
            if size >= n:
                return size if not singles or size <= MIXED_GRAPH_TOKENS else 0
        return 0

    def _step_prompt_graph(self, seqs: List[SeqStep], size: int) -> torch.Tensor:
        singles = len(seqs) - 1
        rows = _bucket(singles) if singles else 0
        ctx = build_context(seqs, self.manager, self.buffers, self.model.dtype, self.model.spec.vocab_size,
                            pad_to=rows or None, pad_tokens_to=size)
        if rows:
            ctx.max_context = self.max_seq_len      # as in a recorded decode step: choices that hold for any context
        # what parts choose on the host for this step (a kernel's shape for a short or a long context) is part of
        # the key: a replay runs what the step would run unrecorded
        key = (rows, size, len(seqs[-1].want), self.model.graph_variant(ctx))
        if key not in self._prompt_graphs:
            self._prompt_graphs[key] = self._record(ctx)        # leaves the step's arrays as they are
        graph, out = self._prompt_graphs[key]
        graph.replay()
        if rows > singles:                                       # drop the rows of the padding
            out = torch.cat([out[:singles], out[rows:]])
        return out

    def _capture(self, size: int, seqs: List[SeqStep]) -> None:
        ctx = build_context(seqs, self.manager, self.buffers, self.model.dtype, self.model.spec.vocab_size,
                            pad_to=size)
        ctx.max_context = self.max_seq_len          # kernel choices must hold for every later replay
        self._graphs[size] = self._record(ctx)

    def _record(self, ctx) -> tuple:
        """Warm up on the real batch, then record the graph.  The warm-up runs write this step's keys and
        values, which the replay that follows writes again with the same values; per-request state, which
        a run changes from what it was, is put back afterwards so that only the replay counts."""
        saved = self.storage.save_state()
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                self.model.forward(ctx, self.storage)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, pool=self._graph_pool):
            out = self.model.forward(ctx, self.storage)
        self.storage.restore_state(saved)
        return graph, out

    # ---- sizes for reports ----------------------------------------------
    def decode_bytes(self, context_lens: List[int]) -> int:
        """Bytes a decode step has to read: every weight once and the cache of the live requests."""
        return self.model.num_weight_bytes() + self.storage.bytes_per_token() * sum(context_lens)
