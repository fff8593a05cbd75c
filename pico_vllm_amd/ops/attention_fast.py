"""The matrix-core attention kernels of the bfloat16 engine and the choice between them."""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import library
from .kernels import KernelError, _check, _check_cache, _ptr, _stream

c_float = ctypes.c_float


_cus = {}


def compute_units(device: int = 0) -> int:
    """Compute units of the GPU, asked once (256 on an MI355X); the cost models below count workgroups against it."""
    if device not in _cus:
        _cus[device] = torch.cuda.get_device_properties(device).multi_processor_count if torch.cuda.is_available() else 256
    return _cus[device]


def supported(nq: int, nkv: int, head_dim: int, window: int) -> bool:
    """Head sizes in steps of 16 up to 256, with or without a window; anything else goes to the plain kernel."""
    return head_dim % 16 == 0 and 16 <= head_dim <= 256 and 0 <= window < (1 << 30) and nq % nkv == 0


class FastAttention:
    def __init__(self, nq: int, nkv: int, head_dim: int, window: int = 0):
        self.nq, self.nkv, self.d, self.window = nq, nkv, head_dim, window
        self.lib = library.attention_library(head_dim)
        if self.lib.pico_attn_head_dim() != head_dim:
            raise KernelError("attention library was built for another head size")
        self.cus = compute_units()

    def num_splits(self, num_seqs: int, max_context: int) -> int:
        """Enough workgroups to fill the chip (two workgroups a compute unit), no split shorter
        than one 64-key tile (or, beyond 64 splits, than two), at most 256 splits (what the merging kernel takes):
        a single request with 32,768 tokens behind it is read by 512 workgroups, not by 128."""
        # the number of sequences counts as the power of two that a recorded step of them is padded to, so that
        # a step splits its contexts alike whether it is replayed from a graph or not
        padded = self.padded(num_seqs)
        by_fill = max(1, 2 * self.cus // max(1, padded * self.nkv))
        keys = min(max_context, self.window + 31) if self.window else max_context      # what a query reads at most
        by_len = max(1, -(-keys // 64))
        if by_len > 64:
            by_len = max(64, -(-keys // 128))
        return max(1, min(by_fill, by_len, 256))

    @staticmethod
    def padded(num_seqs: int) -> int:
        """The power of two that a recorded decode step of so many sequences is padded to."""
        padded = 1
        while padded < num_seqs:
            padded *= 2
        return padded

    CUT_FROM = 32       # sequences (padded) from which a decode step's contexts are cut into pieces of one length

    def decode_cut(self, num_seqs: int, nsplit: int, device) -> Optional[tuple]:
        """Room for the cut of a decode step's contexts into pieces of one length over all sequences (``decode(cut=...)``),
        or None where every sequence keeps ``nsplit`` splits of its own: few sequences (unequal contexts cost
        nothing there: 15.3 against 14.9 us at 8 sequences, 16.1 against 16.1 at 16, but 22.6 against 18.2 at 32 and
        35 against 27 at 64, while the cut's indirection costs a layer about 1 us) or a single split.  The pieces
        fill the workgroups that ``nsplit`` splits of the padded number of sequences would."""
        padded = self.padded(num_seqs)
        if nsplit < 2 or padded < self.CUT_FROM or num_seqs > 1024:
            return None
        slots = padded * nsplit
        return torch.empty(4 * slots + 2 * num_seqs, dtype=torch.int32, device=device), slots

    def prefill_teams(self, new_lens, context_lens) -> int:
        """The shape of the prefill workgroups.  1 to 3: teams of four waves that share the key loop of a
        64-query tile; three cut the longest workgroup's loop to a third, which decides while the work (in
        64 x 64 tiles) would not keep 256 compute units busy for the time the longest tile takes (41 us
        against 43 with two teams and 52 with one for 2,048 tokens of 12 heads); one leaves room for three
        workgroups per unit, which serves many long tiles best (214 against 308 us for eight such prompts).
        4: one team whose waves own two blocks of 16 queries, 128 queries a workgroup: half the LDS traffic
        per product, which is the bound when every compute unit has plenty to do (184 us for the eight
        prompts, 622 against 825 us for four portions of 2,048 tokens after 2,048 with 40 heads), but coarser
        tiles, so only for much work in portions that fill them.
        6: such waves in two teams (eight waves a workgroup): between the two, when there is more than the longest
        tile's worth of work for every unit but not 64 tiles' worth (two prompts of 2,048 tokens of 12 heads: 56 us
        against 71 with 4 and 74 with 1; one prompt of 28 heads: 63 against 71 and 72; four portions of 512 after
        512: 32 against 36 and 39)."""
        longest, total, tokens, padded = 1, 0, 0, 0
        window = getattr(self, "window", 0)
        for n, c in zip(new_lens, context_lens):
            n, c = int(n), int(c)
            if window:
                c = min(c, window + n)                    # the keys that the portion's queries still see
            tiles = -(-n // 64)
            longest = max(longest, -(-c // 64))
            total += tiles * max(1, (2 * c - n) // 128)      # mean key tiles of the portion's query tiles
            tokens += n
            padded += -(-n // 128) * 128
        cus = getattr(self, "cus", None) or compute_units()
        if total * self.nq < cus * longest:
            return 3
        if 4 * tokens < 3 * padded:
            return 1
        return 4 if total * self.nq >= cus * 64 else 6

    def prefill_chunks(self, new_lens, context_lens):
        """(shape, chunk_len, max_chunks) when the keys of the query tiles are better cut into chunks that run as
        workgroups of their own and are joined by a second launch, or None.  That pays where whole tiles leave
        compute units idle or a last round of workgroups nearly empty: portions behind a long prefix with few
        heads or few query tiles (2,048 tokens of 12 heads after 14,336: 341 against 539 us; of 40 heads after
        30,720: 1.70 against 2.20 ms; 512 tokens of 12 heads after 7,680: 69 against 133 us), and not where there
        is work for every unit anyway (28 heads: no gain) or no prefix (the causal triangle's tiles are short).
        The cost of a cut into S chunks is counted in passes of a workgroup over all keys: rounds of workgroups
        over the chip's places, each 1/S long, plus what the partial results cost to write, read and join (with 8
        chunks of 2,048 tokens of 12 heads the second launch reads 104 MB and takes 25 us)."""
        if self.window or self.d % 32:
            return None
        tokens = int(sum(int(n) for n in new_lens))
        keys = int(sum(int(c) for c in context_lens))
        longest = max(int(c) for c in context_lens)
        if keys - tokens < tokens or longest < 2048:               # the prefix is the smaller part of the work, or short
            return None
        padded = sum(-(-int(n) // 128) * 128 for n in new_lens)
        shape = 4 if 4 * tokens >= 3 * padded else 1               # 128-query tiles where the portions fill them
        per_tile, resident = (128, 2) if shape == 4 else (64, 3)
        workgroups = sum(-(-int(n) // per_tile) for n in new_lens) * self.nq
        places = self.cus * resident
        # whole tiles: rounds of workgroups, the last one as good as full when the tiles' lengths differ (long ones
        # start first and short ones fill the gaps), nearly empty when the prefix makes them all alike
        rounds, alike = workgroups / places, (keys - tokens) / keys
        whole = max(1.0, rounds + alike * (-(-workgroups // places) - rounds))
        best, choice = 0.8 * whole, None
        for want in (2, 4, 8, 16):
            chunk_len = 512
            while chunk_len * want < longest:
                chunk_len *= 2                                     # powers of two: few different recorded steps
            chunks = -(-longest // chunk_len)
            if chunks < 2:
                continue
            cost = -(-workgroups * chunks // places) / chunks + 8.0 * chunks / (longest / 64)
            if cost < best:
                best, choice = cost, (shape, chunk_len, want)
        return choice

    def prefill(self, q: torch.Tensor, k_cache, v_cache, block_table, cu_seqlens, context_lens, num_seqs: int,
                scale: float, out: Optional[torch.Tensor] = None, teams: int = 0, chunk_len: int = 0,
                max_chunks: int = 0, order: Optional[torch.Tensor] = None, order_build: bool = True) -> torch.Tensor:
        """q [T, >= nq*d] bfloat16 (row stride free); any mixture of portions; returns [T, nq*d].
        teams: 0 lets the kernel choose, else the result of ``prefill_teams``.  chunk_len > 0: the keys of every
        query tile are cut into chunks of that many, each a workgroup of its own (``max_chunks`` of them cover the
        longest context), and a second launch joins them.  order: ``order_list(T, num_seqs)``, where the kernel
        writes (``order_build``) or finds (the other layers of a step) the query tiles of all sequences longest
        first; without it the sequences are taken one after the other."""
        nq, nkv, d = self.nq, self.nkv, self.d
        T = q.shape[0]
        pages, P = _check_cache(k_cache, v_cache, nkv, d)
        self._check_q(q, k_cache)
        self._check_meta(block_table, cu_seqlens, num_seqs + 1, context_lens, num_seqs)
        if out is None:
            out = torch.empty(T, nq * d, dtype=torch.bfloat16, device=q.device)
        part = None
        if chunk_len and k_cache.numel() * k_cache.element_size() >= (1 << 32):
            chunk_len = max_chunks = 0          # the kernel that cuts keys into chunks addresses the cache with 32 bits
        if chunk_len:
            if self.window or d % 32 or max_chunks < 1:
                raise KernelError("chunks of keys: no window, a head size in steps of 32 and at least one chunk")
            part = torch.empty(T * nq * max_chunks * (d + 4), dtype=torch.float32, device=q.device)
        _check(self.lib, self.lib.pico_attn_prefill(
            _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1],
            _ptr(cu_seqlens), _ptr(context_lens), num_seqs, T, _ptr(out), nq, nkv, d, P, pages, c_float(scale),
            teams, self.window, chunk_len, max_chunks, _ptr(part), _ptr(order), 0 if order is None else order.numel(),
            1 if order_build else 0, _stream()))
        return out

    @staticmethod
    def order_list(num_tokens: int, num_seqs: int, device) -> torch.Tensor:
        """Room for the list of a step's query tiles (``prefill(order=...)``): one entry a tile of 64 queries at most."""
        return torch.empty(num_tokens // 64 + num_seqs, dtype=torch.int32, device=device)

    def decode(self, q: torch.Tensor, k_cache, v_cache, block_table, context_lens, num_seqs: int, scale: float,
               nsplit: int, out: Optional[torch.Tensor] = None, cut: Optional[tuple] = None,
               cut_build: bool = True) -> torch.Tensor:
        """One query token per sequence: q [B, >= nq*d]; returns [B, nq*d].  cut: ``decode_cut(...)``, where the
        kernel writes (``cut_build``) or finds (the other layers of a step) the pieces of one length that the contexts
        of all sequences are cut into; without it every sequence is cut into ``nsplit`` splits of its own."""
        nq, nkv, d = self.nq, self.nkv, self.d
        if q.shape[0] != num_seqs:
            raise KernelError("decode attention wants exactly one query token per sequence")
        if nq // nkv > 32:
            raise KernelError("decode attention handles at most 32 query heads per kv head")
        pages, P = _check_cache(k_cache, v_cache, nkv, d)
        self._check_q(q, k_cache)
        self._check_meta(block_table, None, 0, context_lens, num_seqs)
        if out is None:
            out = torch.empty(num_seqs, nq * d, dtype=torch.bfloat16, device=q.device)
        plan, slots = cut if cut is not None else (None, 0)
        part = torch.empty(max(num_seqs * nsplit, slots) * nq * (d + 2), dtype=torch.float32, device=q.device)
        _check(self.lib, self.lib.pico_attn_decode(
            _ptr(q), q.stride(0), _ptr(k_cache), _ptr(v_cache), _ptr(block_table), block_table.shape[1],
            _ptr(context_lens), num_seqs, _ptr(out), _ptr(part), nsplit, nq, nkv, d, P, pages, c_float(scale),
            self.window, _ptr(plan), slots, 1 if cut_build else 0, _stream()))
        return out

    def _step_cut(self, ctx, num_seqs: int, nsplit: int, device):
        """(cut, build) of a step's decoding sequences: written by the first layer that asks, found by the others."""
        key = ("fast_attention_cut", self.nq, self.nkv, self.d, self.window, num_seqs, nsplit)
        if key in ctx.shared:
            return ctx.shared[key], False
        cut = ctx.shared[key] = self.decode_cut(num_seqs, nsplit, device)
        return cut, True

    def _check_q(self, q, k_cache):
        if not q.is_cuda or q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16:
            raise KernelError("matrix-core attention wants bfloat16 tensors on the GPU")
        if q.dim() != 2 or q.stride(1) != 1 or q.shape[1] < self.nq * self.d:
            raise KernelError("q must be [T, >= nq*d] with unit stride along the row")

    @staticmethod
    def _check_meta(block_table, cu_seqlens, n_cu, context_lens, num_seqs):
        if block_table.dtype != torch.int32 or block_table.dim() != 2 or not block_table.is_contiguous() \
                or block_table.shape[0] < num_seqs:
            raise KernelError("block_table must be contiguous int32 [sequences, pages]")
        for t, n in ((cu_seqlens, n_cu), (context_lens, num_seqs)):
            if t is not None and (t.dtype != torch.int32 or t.numel() < n or not t.is_contiguous()):
                raise KernelError("sequence metadata must be contiguous int32")

    def plan(self, ctx) -> tuple:
        """(teams, lead, chunk_len, max_chunks) of a step with prompt portions: the shape of the prefill workgroups,
        how many single tokens stand first, and into what chunks the keys are cut (0, 0: whole).  Decided on the host
        from the shape of the batch, once for every layer of the step."""
        key = ("fast_attention", self.nq, self.nkv, self.d, self.window)
        if key not in ctx.shared:
            B = ctx.num_seqs
            teams, lead, chunk_len, max_chunks = 0, 0, 0, 0
            if "cu_seqlens" in ctx.host and "context_lens" in ctx.host:
                cu = ctx.host["cu_seqlens"]
                lens = cu[1:B + 1] - cu[:B]
                # the filler behind a recorded step's portion does not count: the step gets the shapes it would get
                # unrecorded, and so the same bits
                real = B - int(ctx.host.get("filler", 0))
                while lead < real and lens[lead] == 1:
                    lead += 1
                if lead < real:
                    teams = self.prefill_teams(lens[lead:real], ctx.host["context_lens"][lead:real])
                    cut = self.prefill_chunks(lens[lead:real], ctx.host["context_lens"][lead:real])
                    if cut is not None:
                        teams, chunk_len, max_chunks = cut
            ctx.shared[key] = (int(teams), int(lead), int(chunk_len), int(max_chunks))
        return ctx.shared[key]

    def __call__(self, qkv, cache, block_table, ctx, scale):
        B = ctx.num_seqs
        grouped = self.nq // self.nkv <= 32
        if ctx.all_decode and grouped:
            nsplit = self.num_splits(B, ctx.max_context)
            cut, build = self._step_cut(ctx, B, nsplit, qkv.device)
            return self.decode(qkv, cache.k, cache.v, block_table, ctx.context_lens, B, scale, nsplit, cut=cut, cut_build=build)
        teams, lead, chunk_len, max_chunks = self.plan(ctx)
        if not grouped:
            lead = 0
        # several portions: the list of their query tiles, longest first, written by the first layer of the step
        order, build = None, False
        if B - lead >= 2:
            key = ("fast_attention_order", self.d, teams, lead)        # the tiles' size goes with the head size and the shape
            order, build = ctx.shared.get(key), key not in ctx.shared
            if build:
                order = ctx.shared[key] = self.order_list(qkv.shape[0], B - lead, qkv.device)
        if lead == 0:
            return self.prefill(qkv, cache.k, cache.v, block_table, ctx.cu_seqlens, ctx.context_lens, B, scale, teams=teams,
                                chunk_len=chunk_len, max_chunks=max_chunks, order=order, order_build=build)
        # A mixed step: the scheduler puts the decoding requests first.  Their tokens (one row each, rows
        # 0 .. lead - 1) go through the decode kernel, which reads keys and values once for all query heads of
        # a group; the prompt portions behind them through the prefill kernel, whose offsets are absolute.
        out = torch.empty(qkv.shape[0], self.nq * self.d, dtype=torch.bfloat16, device=qkv.device)
        nsplit = self.num_splits(lead, ctx.max_context)
        cut, cut_build = self._step_cut(ctx, lead, nsplit, qkv.device)
        self.decode(qkv[:lead], cache.k, cache.v, block_table[:lead], ctx.context_lens[:lead], lead, scale, nsplit, out=out[:lead],
                    cut=cut, cut_build=cut_build)
        if lead < B:
            self.prefill(qkv, cache.k, cache.v, block_table[lead:], ctx.cu_seqlens[lead:], ctx.context_lens[lead:],
                         B - lead, scale, out=out, teams=teams, chunk_len=chunk_len, max_chunks=max_chunks, order=order,
                         order_build=build)
        return out


def choose(nq: int, nkv: int, head_dim: int, window: int) -> Optional[FastAttention]:
    """The matrix-core kernels for these sizes, or None when they are outside what the kernels
    take (the plain kernel then serves them)."""
    if not supported(nq, nkv, head_dim, window):
        return None
    return FastAttention(nq, nkv, head_dim, window)
