"""One step's batch: from (request, its next tokens, wanted places) on the host
to the flat arrays on the device that the parts read.

All integer arrays of a step travel in one pinned buffer and one copy.  The
reference builds five tensors per decode step from Python lists and refills a
[B, 8192] block table (pico_vllm/engine.py:146-181,198-220).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..parts.base import StepContext


@dataclass
class SeqStep:
    """One request's share of a step: its next ``tokens`` (they follow the
    ``num_cached`` tokens already in the cache) and ``want``, the places among
    these tokens whose logits are asked for."""
    req: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


class BatchError(ValueError):
    pass


class BatchBuffers:
    """Pinned host and device int32 buffers of fixed capacity, reused every step."""

    def __init__(self, device: torch.device, max_tokens: int, max_seqs: int, max_pages: int, num_groups: int,
                 max_want: Optional[int] = None):
        self.device = device
        self.max_tokens, self.max_seqs, self.max_pages, self.num_groups = max_tokens, max_seqs, max_pages, num_groups
        self.max_want = max_want if max_want is not None else max_tokens
        n = (3 + num_groups) * max_tokens + (max_seqs + 1) + 2 * max_seqs + self.max_want \
            + num_groups * max_seqs * max_pages
        self.host = torch.zeros(n, dtype=torch.int32, pin_memory=torch.cuda.is_available())
        self.dev = torch.zeros(n, dtype=torch.int32, device=device)
        self.copied = torch.cuda.Event() if torch.cuda.is_available() else None


def build_context(seqs: List[SeqStep], manager: CacheManager, buf: BatchBuffers, act_dtype: torch.dtype,
                  vocab_size: int, pad_to: Optional[int] = None, pad_tokens_to: Optional[int] = None) -> StepContext:
    """Pack ``seqs`` into ``buf`` and describe the device views.

    ``pad_to``: pad a pure-decode batch with empty rows up to that many
    sequences (for replaying a graph captured at that size); a padded row has a
    block table of -1 and a context of 0, so nothing is written for it, its state slot is
    the spare one behind the requests' slots, and its output is ignored.
    ``pad_tokens_to``: bring the step to that many tokens (for replaying a graph of a prompt step
    recorded at that size) with one more sequence of filler tokens behind the given ones: positions
    from 0, a context of its own length, a block table of -1, slots of -1, the spare state slot,
    nothing wanted; it may be empty.
    Both: single-token sequences followed by ONE prompt portion.  The single tokens are padded with empty rows to
    ``pad_to`` of them (the empty rows stand between the real ones and the portion, and are wanted like them), and
    the portion with filler to ``pad_tokens_to`` tokens: ``pad_to + pad_tokens_to`` tokens in ``pad_to + 2`` sequences.
    """
    B = len(seqs)
    if B == 0:
        raise BatchError("a step needs at least one sequence")
    lens = [len(s.tokens) for s in seqs]
    if min(lens) < 1:
        raise BatchError("every sequence of a step brings at least one token")
    if len({s.req for s in seqs}) != B:
        raise BatchError("a request stands twice in one step: its tokens would take the same places in the cache")
    mixed = bool(pad_to) and pad_tokens_to is not None
    filler = 0
    if mixed:
        if max(lens[:-1], default=1) != 1 or pad_to < B - 1:
            raise BatchError(f"a step padded both ways is single tokens (at most {pad_to}) followed by one prompt portion")
        filler = pad_tokens_to - lens[-1]
        empty = pad_to - (B - 1)
        rows = pad_to + 2
        T = pad_to + pad_tokens_to
    elif pad_tokens_to is not None:
        filler = pad_tokens_to - sum(lens)
        empty = 0
        rows = B + 1
        T = pad_tokens_to
    else:
        rows = max(B, pad_to or 0)
        empty = rows - B
        T = sum(lens) + empty
    if filler < 0:
        raise BatchError(f"the step has {sum(lens) if not mixed else lens[-1]} tokens, more than the {pad_tokens_to} it is to be padded to")
    R = sum(len(s.want) for s in seqs) + (empty if pad_to else 0)
    P = manager.page_size
    if T > buf.max_tokens or rows > buf.max_seqs or R > buf.max_want:
        raise BatchError(f"step of {T} tokens / {rows} sequences / {R} wanted rows exceeds the buffers "
                         f"({buf.max_tokens} / {buf.max_seqs} / {buf.max_want})")
    G = len(manager.groups)
    if buf.copied is not None:
        buf.copied.synchronize()          # the previous step's copy has left the pinned buffer
    h = buf.host.numpy()
    h_tok, h_pos, h_seq = h[0:T], h[buf.max_tokens:buf.max_tokens + T], h[2 * buf.max_tokens:2 * buf.max_tokens + T]
    h_slots = [h[(3 + g) * buf.max_tokens:(3 + g) * buf.max_tokens + T] for g in range(G)]
    o = (3 + G) * buf.max_tokens
    h_cu = h[o:o + rows + 1]; o += buf.max_seqs + 1
    h_ctx = h[o:o + rows]; o += buf.max_seqs
    h_slot = h[o:o + rows]; o += buf.max_seqs
    h_want = h[o:o + R]; o += buf.max_want
    bt_off = o
    max_ctx = 1
    need_pages = 1
    t = 0
    r = 0
    h_cu[0] = 0
    spare = manager.slots.num_slots                # the state slot that no request ever holds
    # the rows of the step: the given sequences in their order; empty rows behind them, or (padded both ways) in front
    # of the portion that stands last; the filler at the very end
    row_of = list(range(B)) if not mixed else list(range(B - 1)) + [pad_to]

    def empty_rows(first: int, end: int) -> None:
        nonlocal t, r
        for e in range(first, end):
            h_tok[t] = 0; h_pos[t] = 0; h_seq[t] = e
            h_want[r] = t; r += 1
            t += 1
            h_cu[e + 1] = t
            h_ctx[e] = 0
            h_slot[e] = spare

    for b, s in zip(row_of, seqs):
        if mixed and b == pad_to:
            empty_rows(B - 1, pad_to)              # between the single tokens and the portion
        n = len(s.tokens)
        cached = manager.num_computed(s.req)
        if n == 1:
            tok = s.tokens[0]
            if not 0 <= tok < vocab_size:
                raise BatchError(f"request {s.req!r}: token id outside [0, {vocab_size})")
            h_tok[t] = tok
            h_pos[t] = cached
            h_seq[t] = b
            for w in s.want:
                if w != 0:
                    raise BatchError(f"request {s.req!r}: wanted place {w} is outside its 1 tokens")
                h_want[r] = t
                r += 1
            t += 1
            h_cu[b + 1] = t
            h_ctx[b] = cached + 1
            h_slot[b] = manager.slot(s.req)
            max_ctx = max(max_ctx, cached + 1)
            need_pages = max(need_pages, -(-(cached + 1) // P))
            continue
        toks = np.asarray(s.tokens, dtype=np.int64)
        if toks.min() < 0 or toks.max() >= vocab_size:
            raise BatchError(f"request {s.req!r}: token id outside [0, {vocab_size})")
        h_tok[t:t + n] = toks
        h_pos[t:t + n] = np.arange(cached, cached + n)
        h_seq[t:t + n] = b
        for w in s.want:
            if not 0 <= w < n:
                raise BatchError(f"request {s.req!r}: wanted place {w} is outside its {n} tokens")
            h_want[r] = t + w
            r += 1
        t += n
        h_cu[b + 1] = t
        h_ctx[b] = cached + n
        h_slot[b] = manager.slot(s.req)
        max_ctx = max(max_ctx, cached + n)
        need_pages = max(need_pages, -(-(cached + n) // P))
    last = row_of[-1] + 1                          # the first row behind the given sequences
    if pad_tokens_to is not None:                  # the sequence of filler tokens of a recorded prompt step
        h_tok[t:T] = 0
        h_pos[t:T] = np.arange(filler)
        h_seq[t:T] = last
        h_cu[last + 1] = T
        h_ctx[last] = filler
        h_slot[last] = spare
    else:
        empty_rows(last, rows)                     # padding rows of a captured decode batch
    width = buf.max_pages if (pad_to or pad_tokens_to is not None) else need_pages
    if width > buf.max_pages:
        raise BatchError(f"a sequence needs {width} pages, the buffers hold {buf.max_pages} per sequence")
    tables = h[bt_off:bt_off + G * rows * width].reshape(G, rows, width)
    tables[:] = -1
    if rows > B:
        for g in range(G):
            h_slots[g][:] = -1                                          # padding rows and filler store nothing
    for b, s in zip(row_of, seqs):
        need = -(-int(h_ctx[b]) // P)
        lo, hi = int(h_cu[b]), int(h_cu[b + 1])
        for g in range(G):
            table = manager.block_table_array(s.req, g, need)
            tables[g, b, :need] = table
            pos = h_pos[lo:hi]
            h_slots[g][lo:hi] = table[pos // P] * P + pos % P          # pico_vllm/cache.py:143-156
    used = bt_off + G * rows * width
    buf.dev[:used].copy_(buf.host[:used], non_blocking=True)
    if buf.copied is not None:
        buf.copied.record()
    d = buf.dev
    o = (3 + G) * buf.max_tokens
    ctx = StepContext(
        num_tokens=T, num_seqs=rows,
        token_ids=d[0:T], positions=d[buf.max_tokens:buf.max_tokens + T],
        token_seq=d[2 * buf.max_tokens:2 * buf.max_tokens + T],
        cu_seqlens=d[o:o + rows + 1],
        context_lens=d[o + buf.max_seqs + 1:o + buf.max_seqs + 1 + rows],
        state_slots=d[o + 2 * buf.max_seqs + 1:o + 2 * buf.max_seqs + 1 + rows],
        want_rows=d[o + 3 * buf.max_seqs + 1:o + 3 * buf.max_seqs + 1 + R],
        block_tables=[d[bt_off + g * rows * width:bt_off + (g + 1) * rows * width].view(rows, width) for g in range(G)],
        slot_mapping=[d[(3 + g) * buf.max_tokens:(3 + g) * buf.max_tokens + T] for g in range(G)],
        act_dtype=act_dtype,
        max_new_tokens=max(lens), max_context=max_ctx, all_decode=max(lens) == 1 and pad_tokens_to is None,
        # (filler: how many sequences at the end are padding of a recorded step, whose size says nothing about the work)
        host={"cu_seqlens": h_cu.copy(), "context_lens": h_ctx.copy(), "filler": int(pad_tokens_to is not None)},
    )
    return ctx
