"""Page ids with reference counts, and slots for fixed-size state.

The counterpart in the reference is BlockManager's allocator half
(pico_vllm/blockmanager.py:70-133): a free deque, a count per page set to 1
by allocate, inc_ref / dec_ref that frees at zero.  Differences: allocation
reports failure instead of raising from inside a step (blockmanager.py:77-78),
there is no CPU tier, and giving back a page that is not held is an error.
Like there (set_evict_callback, blockmanager.py:66-75) a holder of pages that
it can do without (an index of shared prefixes, say) may register a callable
that is asked to give pages back before an allocation is refused.
"""
from __future__ import annotations

from collections import deque
from typing import Callable, List, Optional


class PagePoolError(RuntimeError):
    pass


class PagePool:
    def __init__(self, num_pages: int):
        if num_pages < 1:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = num_pages
        self._free = deque(range(num_pages))
        self._refs = [0] * num_pages
        self.peak_used = 0
        self.reuse_count = 0           # pages handed out that had been used before
        self._ever_used = [False] * num_pages
        self._reclaim: Optional[Callable[[int], int]] = None

    def set_reclaim_callback(self, cb: Optional[Callable[[int], int]]) -> None:
        """``cb(n)`` is called when ``n`` more pages are wanted than are free; it releases
        pages that it holds (through ``release``) and returns how many holders it dropped,
        0 when it has nothing left to give."""
        self._reclaim = cb

    def ensure_free(self, n: int) -> bool:
        """Whether ``n`` pages are free, after asking the reclaim callback for the difference."""
        while n > len(self._free) and self._reclaim is not None:
            if self._reclaim(n - len(self._free)) <= 0:
                break
        return n <= len(self._free)

    @property
    def num_free(self) -> int:
        return len(self._free)

    @property
    def num_used(self) -> int:
        return self.num_pages - len(self._free)

    def ref_count(self, page: int) -> int:
        return self._refs[page]

    def allocate(self, n: int) -> Optional[List[int]]:
        """n fresh pages with count 1 each, or None (and nothing taken) if fewer are free."""
        if n < 0:
            raise ValueError("cannot allocate a negative number of pages")
        if not self.ensure_free(n):
            return None
        out = [self._free.popleft() for _ in range(n)]
        for p in out:
            self._refs[p] = 1
            self.reuse_count += self._ever_used[p]
            self._ever_used[p] = True
        self.peak_used = max(self.peak_used, self.num_used)
        return out

    def share(self, pages: List[int]) -> None:
        """One more holder for each page (pages must be held already)."""
        for p in pages:
            if self._refs[p] < 1:
                raise PagePoolError(f"page {p} is not held and cannot be shared")
        for p in pages:
            self._refs[p] += 1

    def release(self, pages: List[int]) -> None:
        """One holder fewer for each page; a page nobody holds goes back to the free list."""
        for p in pages:
            if not 0 <= p < self.num_pages or self._refs[p] < 1:
                raise PagePoolError(f"page {p} is given back but is not held")
            self._refs[p] -= 1
            if self._refs[p] == 0:
                self._free.append(p)

    def check(self) -> None:
        free = set(self._free)
        if len(free) != len(self._free):
            raise PagePoolError("a page is on the free list twice")
        for p in range(self.num_pages):
            if (self._refs[p] == 0) != (p in free):
                raise PagePoolError(f"page {p}: count {self._refs[p]} disagrees with the free list")


class StateSlots:
    """``num_slots`` slots of per-request state of fixed size; a request holds
    one from admission to its end, whether or not a layer of the model uses it."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free = deque(range(num_slots))
        self._held = set()

    @property
    def num_free(self) -> int:
        return len(self._free)

    def acquire(self) -> Optional[int]:
        if not self._free:
            return None
        s = self._free.popleft()
        self._held.add(s)
        return s

    def release(self, slot: int) -> None:
        if slot not in self._held:
            raise PagePoolError(f"state slot {slot} is given back but is not held")
        self._held.remove(slot)
        self._free.append(slot)
