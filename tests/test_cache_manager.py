"""The cache manager on the host: pages, block tables, windows, state slots (no GPU)."""
import random

import pytest

from pico_vllm_amd.cache.manager import CacheManager
from pico_vllm_amd.cache.page_pool import PagePool, PagePoolError, StateSlots
from pico_vllm_amd.parts.attention import kv_page_tensors
from pico_vllm_amd.parts.spec import CacheSpec

FULL = CacheSpec("paged_kv", page_tensors=kv_page_tensors(2, 16))
WIN = CacheSpec("paged_kv", window=20, page_tensors=kv_page_tensors(2, 16))
STATE = CacheSpec("state", state_shape=(4,))


def test_pool_allocates_shares_releases_and_refuses_double_free():
    p = PagePool(4)
    a = p.allocate(3)
    assert len(set(a)) == 3 and p.num_free == 1 and all(p.ref_count(x) == 1 for x in a)
    assert p.allocate(2) is None and p.num_free == 1            # nothing taken on failure
    p.share(a[:1])
    p.release(a)                                                # a[0] still held once
    assert p.num_free == 3 and p.ref_count(a[0]) == 1
    p.release(a[:1])
    assert p.num_free == 4
    with pytest.raises(PagePoolError):
        p.release(a[:1])
    with pytest.raises(PagePoolError):
        p.share([a[1]])
    p.check()


def test_freed_pages_are_handed_out_again():
    # as in the reference's 4-page scenario (tests/test_evict_recompute.py:185-226)
    p = PagePool(4)
    a = p.allocate(4)
    assert p.allocate(1) is None
    p.release(a[1:3])
    b = p.allocate(2)
    assert sorted(b) == sorted(a[1:3]) and p.reuse_count == 2


def test_groups_are_formed_by_equal_needs():
    m = CacheManager({0: FULL, 1: WIN, 2: FULL, 3: STATE, 4: WIN, 5: CacheSpec("none")}, 8, 10, 2)
    assert [g.layers for g in m.groups] == [[0, 2], [1, 4]]
    assert m.layer_group == {0: 0, 2: 0, 1: 1, 4: 1} and m.state_layers == [3]


def test_growth_arithmetic_and_slots():
    m = CacheManager({0: FULL}, 16, 8, 2)
    assert m.add_request("a") and m.add_request("b")
    assert not m.add_request("c")                               # no third state slot
    assert m.slot("a") != m.slot("b")
    assert m.pages_needed("a", 17) == [2]
    assert m.grow("a", 17) and len(m.block_table("a")) == 2
    assert m.grow("a", 32) and len(m.block_table("a")) == 2     # ceil(32/16) = 2: no new page
    assert m.grow("a", 33) and len(m.block_table("a")) == 3
    # slot = page * size + pos % size (pico_vllm/cache.py:132-141)
    assert m.token_slot("a", 18) == m.block_table("a")[1] * 16 + 2
    assert not m.grow("b", 16 * 6)                              # 6 pages wanted, 5 free: nothing changes
    assert m.block_table("b") == [] and m.groups[0].pool.num_free == 5
    m.free_request("a")
    assert m.groups[0].pool.num_free == 8 and m.add_request("c")
    m.check()


def test_window_gives_pages_back_once_passed():
    m = CacheManager({0: FULL, 1: WIN}, 8, 16, 1)
    m.add_request("r")
    assert m.grow("r", 64)
    m.advance("r", 64)
    full, win = m.block_table("r", 0), m.block_table("r", 1)
    assert all(p >= 0 for p in full)
    # next query at position 64 reads keys > 64 - 20 = 44, i.e. from 45: pages 0..4 (positions < 40) are dead
    assert [p < 0 for p in win] == [True] * 5 + [False] * 3
    assert m.groups[1].pool.num_free == 16 - 3 and m.groups[0].pool.num_free == 8
    with pytest.raises(PagePoolError):
        m.token_slot("r", 10, group=1)
    m.check()
    m.free_request("r")
    assert m.groups[1].pool.num_free == 16
    m.check()


def test_prefix_sharing_counts():
    m = CacheManager({0: FULL}, 16, 8, 3)
    m.add_request("a"); m.grow("a", 40); m.advance("a", 40)
    m.add_request("b")
    m.fork_prefix("a", "b", 32)
    assert m.block_table("b") == m.block_table("a")[:2] and m.num_computed("b") == 32
    m.check()
    m.free_request("a")
    assert m.groups[0].pool.num_free == 8 - 2                    # b still holds the two shared pages
    m.free_request("b")
    assert m.groups[0].pool.num_free == 8
    with pytest.raises(ValueError):
        m.add_request("c"); m.add_request("d"); m.grow("c", 20); m.advance("c", 20); m.fork_prefix("c", "d", 20)


def test_a_holder_of_spare_pages_is_asked_before_an_allocation_is_refused():
    """The seam for an index of shared prefixes: it keeps finished requests' pages and gives
    them back, oldest first, when the pool runs short (the reference's evict callback,
    pico_vllm/blockmanager.py:66-75, scenario of tests/test_evict_recompute.py:185-226)."""
    m = CacheManager({0: FULL}, 16, 4, 3)
    pool = m.groups[0].pool
    kept, asked = [], []

    def reclaim(n):
        asked.append(n)
        gone = kept[:n]
        del kept[:n]
        pool.release(gone)
        return len(gone)

    pool.set_reclaim_callback(reclaim)
    m.add_request("a"); assert m.grow("a", 48); m.advance("a", 48)
    pages = list(m.block_table("a"))
    pool.share(pages[:2]); kept.extend(pages[:2])         # the keeper holds a's first two pages
    m.free_request("a")
    assert pool.num_free == 2 and not asked
    m.check([{p: 1 for p in kept}])
    m.add_request("b"); assert m.grow("b", 32) and not asked            # fits without asking
    m.add_request("c"); assert m.grow("c", 16) and asked == [1]         # one page short: the keeper gives its oldest
    assert kept == pages[1:2] and m.block_table("c") == [pages[0]]
    m.check([{p: 1 for p in kept}])
    assert not m.grow("c", 48) and kept == []                           # asked again, gave its last, still short: nothing taken
    assert m.grow("c", 32)
    m.check()
    assert not m.grow("b", 48) and asked[-1] == 1                       # nothing left to give: refused, nothing taken
    m.check()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_never_lose_or_double_hold_a_page(seed):
    rng = random.Random(seed)
    m = CacheManager({0: FULL, 1: WIN, 2: STATE}, 8, 24, 4)
    live = {}
    next_id = 0
    for _ in range(400):
        op = rng.random()
        if op < 0.25 and len(live) < 6:
            rid = f"r{next_id}"; next_id += 1
            if m.add_request(rid):
                live[rid] = 0
            else:
                assert len(live) >= 4
        elif op < 0.8 and live:
            rid = rng.choice(list(live))
            new_len = live[rid] + rng.randint(1, 30)
            free_before = [g.pool.num_free for g in m.groups]
            if m.grow(rid, new_len):
                live[rid] = new_len
                m.advance(rid, new_len)
            else:
                assert [g.pool.num_free for g in m.groups] == free_before      # all or nothing
        elif live:
            rid = rng.choice(list(live))
            m.free_request(rid)
            del live[rid]
        m.check()
    for rid in list(live):
        m.free_request(rid)
    m.check()
    assert all(g.pool.num_free == g.pool.num_pages for g in m.groups) and m.slots.num_free == 4
    assert m.groups[0].pool.reuse_count > 0


def test_state_slots():
    s = StateSlots(2)
    a, b = s.acquire(), s.acquire()
    assert {a, b} == {0, 1} and s.acquire() is None
    s.release(a)
    assert s.acquire() == a
    with pytest.raises(PagePoolError):
        s.release(5)


def test_a_slot_taken_by_a_new_request_is_reported_for_clearing():
    # a state slot is handed out as the last holder left it; the manager tells the owner of the tensors which
    # slots new requests took, once, so that no mixer has to find out by itself that a request is new
    m = CacheManager({0: FULL, 1: STATE}, 16, 8, 2)
    assert m.add_request("a") and m.add_request("b")
    assert sorted(m.take_fresh_slots()) == [0, 1] and m.take_fresh_slots() == []
    m.free_request("a")
    assert m.add_request("c") and m.take_fresh_slots() == [m.slot("c")]
    # a model without state has nothing to clear
    plain = CacheManager({0: FULL}, 16, 8, 2)
    assert plain.add_request("a") and plain.take_fresh_slots() == []


def test_a_model_with_state_cannot_share_a_prefix():
    m = CacheManager({0: FULL, 1: STATE}, 16, 8, 2)
    m.add_request("a")
    assert m.grow("a", 32)
    m.advance("a", 32)
    m.add_request("b")
    with pytest.raises(PagePoolError, match="state"):
        m.fork_prefix("a", "b", 16)
    m.check()


def test_the_checks_find_every_kind_of_damage():
    # the tests above trust PagePool.check and CacheManager.check: each kind of damage, done by hand, is found
    def damaged():
        m = CacheManager({0: FULL, 1: WIN}, 8, 12, 3)
        for r, n in (("a", 30), ("b", 9)):
            m.add_request(r); m.grow(r, n); m.advance(r, n)
        m.check()
        return m

    m = damaged()
    m.groups[0].pool._free.append(m.groups[0].pool._free[0])             # a page twice on the free list
    with pytest.raises(PagePoolError, match="free list twice"):
        m.check()
    m = damaged()
    m.groups[0].pool._free.append(m.block_table("a")[0])                 # a held page that is also free
    with pytest.raises(PagePoolError, match="disagrees with the free list"):
        m.check()
    m = damaged()
    m.groups[0].pool._free.popleft()                                     # a page lost: neither free nor held
    with pytest.raises(PagePoolError, match="disagrees with the free list"):
        m.check()
    m = damaged()
    m.block_table("a")[1] = m.block_table("a")[0]                        # one page twice in a table
    with pytest.raises(PagePoolError, match="twice in one table"):
        m.check()
    m = damaged()
    m.block_table("b")[0] = m.block_table("a")[0]                        # held by two tables, counted once
    with pytest.raises(PagePoolError, match="held by 2 tables"):
        m.check()
    m = damaged()
    m.groups[0].pool.share(m.block_table("a")[:1])                       # counted twice, held by one table
    with pytest.raises(PagePoolError, match="count 2, held by 1"):
        m.check()
    m.check(other_holders=[{m.block_table("a")[0]: 1}, {}])              # unless another holder is named
    m = damaged()
    m.requests["b"].slot = m.requests["a"].slot                          # a slot held twice
    with pytest.raises(PagePoolError, match="slot is held twice"):
        m.check()
    m = damaged()
    m.free_request("b")
    m.slots._free.pop()                                                  # a slot lost
    with pytest.raises(PagePoolError, match="slot was lost"):
        m.check()


def test_what_the_manager_refuses():
    m = CacheManager({0: FULL, 1: WIN}, 8, 12, 3)
    with pytest.raises(ValueError, match="unknown cache kind"):
        CacheManager({0: CacheSpec("ring")}, 8, 12, 3)
    with pytest.raises(ValueError, match="at least one page"):
        PagePool(0)
    with pytest.raises(ValueError, match="negative"):
        PagePool(2).allocate(-1)
    assert m.add_request("a")
    with pytest.raises(PagePoolError, match="already in the cache"):
        m.add_request("a")
    m.grow("a", 64); m.advance("a", 64)
    assert m.num_free_pages() == min(12 - 8, 12 - 3)                      # of the group that has fewest
    assert list(m.block_table_array("a", 0, 3)) == m.block_table("a")[:3]
    with pytest.raises(PagePoolError, match="9 pages are needed, 8 are allocated"):
        m.block_table_array("a", 0, 9)
    m.add_request("b")
    with pytest.raises(ValueError, match="not computed that many"):
        m.fork_prefix("a", "b", 72)
    with pytest.raises(PagePoolError, match="given back by its window"):
        m.fork_prefix("a", "b", 48)                                       # the window's group has dropped pages 0..4
    assert m.block_table("b", 0) == [] and m.block_table("b", 1) == []    # and nothing was shared before it was refused
    m.check()
    m.grow("b", 3); m.advance("b", 3)
    with pytest.raises(PagePoolError, match="must be empty"):
        m.fork_prefix("a", "b", 8)
    m.check()
