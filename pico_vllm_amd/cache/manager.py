"""The cache manager: which pages and which state slot every request holds.

Layers whose mixers declare equal ``CacheSpec``s form a group; a group has a
page pool of its own and every request has one block table per group (the
list of its page ids by page index; -1 where a window has passed and the page
was given back).  All of it is host bookkeeping with no device code; the
tensors live in ``cache.storage``.

Reference counterparts: the per-request view PagedKVCache
(pico_vllm/cache.py:84-156: page lists, growth arithmetic
ceil((len + n) / page) - held, slot = page * size + pos % size) and the
allocator in blockmanager.py.  The reference has one uniform pool, no windows
and no state slots.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np

from ..parts.spec import CacheSpec
from .page_pool import PagePool, PagePoolError, StateSlots


@dataclass
class CacheGroup:
    spec: CacheSpec
    layers: List[int]
    pool: PagePool

    @property
    def window(self) -> int:
        return self.spec.window


@dataclass
class RequestCache:
    slot: int
    tables: List[List[int]]                  # one per group
    num_computed: int = 0                    # tokens whose keys/state are in the cache
    first_live: List[int] = field(default_factory=list)   # per group: first page index still held
    arrays: List[np.ndarray] = field(default_factory=list)  # per group: the table again as int32 array, for packing


def _mirror(rc: RequestCache, gi: int) -> None:
    """Bring the int32 copy of table ``gi`` up to date after the list changed."""
    table = rc.tables[gi]
    arr = rc.arrays[gi]
    if len(table) > arr.shape[0]:
        arr = np.full(max(2 * arr.shape[0], len(table), 16), -1, dtype=np.int32)
        rc.arrays[gi] = arr
    arr[:len(table)] = table


def _cdiv(a: int, b: int) -> int:
    return -(-a // b)


class CacheManager:
    def __init__(self, layer_specs: Dict[int, CacheSpec], page_size: int, num_pages: int, max_seqs: int):
        self.page_size = page_size
        self.groups: List[CacheGroup] = []
        self.layer_group: Dict[int, int] = {}
        self.state_layers: List[int] = []
        for layer in sorted(layer_specs):
            spec = layer_specs[layer]
            if spec.kind == "paged_kv":
                for gi, g in enumerate(self.groups):
                    if g.spec == spec:
                        g.layers.append(layer)
                        self.layer_group[layer] = gi
                        break
                else:
                    self.layer_group[layer] = len(self.groups)
                    self.groups.append(CacheGroup(spec, [layer], PagePool(num_pages)))
            elif spec.kind == "state":
                self.state_layers.append(layer)
            elif spec.kind != "none":
                raise ValueError(f"layer {layer}: unknown cache kind {spec.kind!r}")
        self.slots = StateSlots(max_seqs)
        self.requests: Dict[Hashable, RequestCache] = {}
        # slots handed out since the storage last cleared any: a request's state starts from zero, whoever held
        # the slot before (``take_fresh_slots``; the step function clears them before the model runs)
        self._fresh_slots: List[int] = []

    # ---- requests -------------------------------------------------------
    def add_request(self, req: Hashable) -> bool:
        """Give ``req`` a state slot and empty tables; False if no slot is free."""
        if req in self.requests:
            raise PagePoolError(f"request {req!r} is already in the cache")
        slot = self.slots.acquire()
        if slot is None:
            return False
        self.requests[req] = RequestCache(slot, [[] for _ in self.groups], 0, [0] * len(self.groups),
                                          [np.full(16, -1, dtype=np.int32) for _ in self.groups])
        if self.state_layers:
            self._fresh_slots.append(slot)
        return True

    def take_fresh_slots(self) -> List[int]:
        """The state slots given to new requests since the last call; whoever owns the state tensors sets them
        to zero before the next step reads them, so that no mixer has to find out by itself that a request is new."""
        out, self._fresh_slots = self._fresh_slots, []
        return out

    def free_request(self, req: Hashable) -> None:
        rc = self.requests.pop(req)
        for g, table in zip(self.groups, rc.tables):
            g.pool.release([p for p in table if p >= 0])
        self.slots.release(rc.slot)

    # ---- growth ---------------------------------------------------------
    def pages_needed(self, req: Hashable, new_len: int) -> List[int]:
        """Per group, pages still to allocate so that positions [0, new_len) are covered
        (pico_vllm/cache.py:114-124)."""
        rc = self.requests[req]
        return [max(0, _cdiv(new_len, self.page_size) - len(t)) for t in rc.tables]

    def grow(self, req: Hashable, new_len: int) -> bool:
        """Cover positions [0, new_len) in every group, or change nothing and return False."""
        need = self.pages_needed(req, new_len)
        if not all(g.pool.ensure_free(n) for n, g in zip(need, self.groups)):
            return False
        rc = self.requests[req]
        for gi, (n, g, table) in enumerate(zip(need, self.groups, rc.tables)):
            if n:
                table.extend(g.pool.allocate(n))
                _mirror(rc, gi)
        return True

    def advance(self, req: Hashable, num_computed: int) -> None:
        """Record that positions [0, num_computed) are cached, and give back
        the pages that every window has passed: the next query sits at
        position num_computed or later and reads keys > position - window."""
        rc = self.requests[req]
        rc.num_computed = num_computed
        for gi, g in enumerate(self.groups):
            if g.window <= 0:
                continue
            first_needed = num_computed - g.window + 1      # lowest key position still readable
            if first_needed <= 0:
                continue
            dead_upto = min(first_needed // self.page_size, len(rc.tables[gi]))
            gone = [rc.tables[gi][j] for j in range(rc.first_live[gi], dead_upto)]
            for j in range(rc.first_live[gi], dead_upto):
                rc.tables[gi][j] = -1
            if gone:
                g.pool.release(gone)
                _mirror(rc, gi)
            rc.first_live[gi] = max(rc.first_live[gi], dead_upto)

    def fork_prefix(self, src: Hashable, dst: Hashable, num_tokens: int) -> None:
        """Let ``dst`` (new, empty) share the full pages that hold the first
        ``num_tokens`` positions of ``src``; shared pages are never written
        again because only full pages are shared (pico_vllm/cache.py:170-192,
        engine.py:265)."""
        if num_tokens % self.page_size:
            raise ValueError("only whole pages can be shared")
        if self.state_layers:
            # a fixed-size state exists only as of the source's last token, not as of the end of the prefix
            raise PagePoolError("a model with per-request state cannot share a prefix: the state at the end of the "
                                "prefix is not kept")
        s, d = self.requests[src], self.requests[dst]
        if d.num_computed or any(d.tables):
            raise PagePoolError("the receiving request must be empty")
        if num_tokens > s.num_computed:
            raise ValueError("the source has not computed that many tokens")
        n = num_tokens // self.page_size
        if any(p < 0 for st in s.tables for p in st[:n]):                # before anything is changed
            raise PagePoolError("a page of the prefix was already given back by its window")
        for g, st, dt in zip(self.groups, s.tables, d.tables):
            g.pool.share(st[:n])
            dt.extend(st[:n])
        for gi in range(len(self.groups)):
            _mirror(d, gi)
        d.num_computed = num_tokens

    # ---- views ----------------------------------------------------------
    def block_table(self, req: Hashable, group: int = 0) -> List[int]:
        return self.requests[req].tables[group]

    def block_table_array(self, req: Hashable, group: int, n: int) -> np.ndarray:
        """The first ``n`` entries of the table as an int32 array (a view; do not write)."""
        rc = self.requests[req]
        if n > len(rc.tables[group]):
            raise PagePoolError(f"request {req!r}: {n} pages are needed, {len(rc.tables[group])} are allocated")
        return rc.arrays[group][:n]

    def slot(self, req: Hashable) -> int:
        return self.requests[req].slot

    def num_computed(self, req: Hashable) -> int:
        return self.requests[req].num_computed

    def num_free_pages(self) -> int:
        return min((g.pool.num_free for g in self.groups), default=1 << 30)

    def token_slot(self, req: Hashable, position: int, group: int = 0) -> int:
        """page * page_size + position % page_size (pico_vllm/cache.py:132-141)."""
        page = self.requests[req].tables[group][position // self.page_size]
        if page < 0:
            raise PagePoolError(f"position {position} of request {req!r} lies on a page that was given back")
        return page * self.page_size + position % self.page_size

    # ---- invariants -----------------------------------------------------
    def check(self, other_holders: Optional[Sequence[Dict[int, int]]] = None) -> None:
        """No page lost, none held more often than counted, none both free and held.
        ``other_holders``: per group, page -> count for holders that are no requests
        (whoever registered a reclaim callback)."""
        for gi, g in enumerate(self.groups):
            g.pool.check()
            holders: Dict[int, int] = dict(other_holders[gi]) if other_holders else {}
            for rc in self.requests.values():
                seen = set()
                for p in rc.tables[gi]:
                    if p < 0:
                        continue
                    if p in seen:
                        raise PagePoolError(f"page {p} appears twice in one table")
                    seen.add(p)
                    holders[p] = holders.get(p, 0) + 1
            for p in range(g.pool.num_pages):
                if g.pool.ref_count(p) != holders.get(p, 0):
                    raise PagePoolError(f"group {gi} page {p}: count {g.pool.ref_count(p)}, "
                                        f"held by {holders.get(p, 0)} tables")
            if g.pool.num_free + len(holders) != g.pool.num_pages:
                raise PagePoolError(f"group {gi}: free + held != total")
        held_slots = sorted(rc.slot for rc in self.requests.values())
        if len(set(held_slots)) != len(held_slots):
            raise PagePoolError("a state slot is held twice")
        if self.slots.num_free + len(held_slots) != self.slots.num_slots:
            raise PagePoolError("a state slot was lost")
