"""The product's page pool (libkvx over accounting-only storage, no GPU needed)
against the reference's pool cases with their exact page ids and moves
(dev/tests/engine/elastic_kv_pool_test.cpp:40-383) -- the same cases
tests/test_oracle_pool.py holds the oracle to.  Page contents are followed on
the device in tests/test_gpu_append.py; here a copy is bookkeeping only."""
import ctypes as C

import pytest

from richengine_amd import kvx

L = kvx.lib()
NO_LIMIT = 0xFFFFFFFF


class Pool:
    def __init__(self, pages, runway, extent_pages=4, budget_pages=None):
        self.storage = kvx.Storage(1, 1, 64, kvx.INT8, pages, extent_pages, accounting=True)
        self.page_bytes = self.storage.bytes_per_page
        self.extent_bytes = self.storage.extent_bytes
        if budget_pages is not None:
            self.budget(budget_pages)
        self.pool = kvx.Pool(self.storage, runway)

    def budget(self, pages):
        # 0 pages: refuse everything (a budget of one byte); None: no budget
        L.kvx_storage_set_budget(self.storage.h, 0 if pages is None else max(1, pages * self.page_bytes))

    def acquire(self, count):
        try:
            return count, self.pool.acquire(count)
        except kvx.KvxError as e:
            return {kvx.ENOMEM: -1, kvx.ESTATE: -2}[e.code], []

    def release(self, pages, prefix=False):
        for p in pages:
            self.pool.release(int(p), prefix)

    def retain(self, page, prefix):
        try:
            self.pool.retain(page, prefix)
            return 0
        except kvx.KvxError:
            return -1

    def snap(self):
        return self.pool.snapshot()

    def reclaim(self, keep, limit=NO_LIMIT):
        return self.pool.reclaim_empty(keep, limit)

    def active(self, page):
        return self.pool.page_active(page)

    def compact(self, fixed=()):
        return self.pool.compact_extent(list(fixed))

    def allocated(self, extent):
        return bool(L.kvx_storage_is_allocated(self.storage.h, extent * self.storage.extent_pages))


def follow(moves, page):
    if moves and moves["first"] <= page < moves["first"] + len(moves["dest"]):
        return moves["dest"][page - moves["first"]]
    return page


def held(pages, released):
    pool = Pool(pages, pages)
    rc, _ = pool.acquire(pages)
    assert rc == pages
    pool.release(released)
    return pool


def test_growth_packs_allocated_extents():
    pool = Pool(12, 4)
    rc, pages = pool.acquire(5)
    assert rc == 5 and pages[0] == 0 and pages[3] == 3 and pages[4] == 4
    s = pool.snap()
    assert (s.pages_allocated, s.pages_active, s.pages_free) == (8, 5, 3)
    assert s.allocated_bytes == 2 * pool.extent_bytes
    pool.release(pages)
    assert pool.reclaim(True) == pool.extent_bytes
    s = pool.snap()
    assert s.pages_allocated == 4 and s.reclaimable_bytes == pool.extent_bytes
    assert s.extent_allocations == 2 and s.extent_releases == 1


def test_runway_is_allocated_through_the_pool():
    pool = Pool(16, 6)
    s = pool.snap()
    assert s.extent_allocations == 2 and s.pages_allocated == 8
    assert s.reclaimable_bytes == 2 * pool.extent_bytes
    assert pool.allocated(0) and pool.allocated(1) and not pool.allocated(2)
    assert pool.reclaim(True) == pool.extent_bytes
    s = pool.snap()
    assert s.extent_allocations - s.extent_releases == 1 and s.pages_allocated == 4
    with pytest.raises(kvx.KvxError) as refused:      # a refused runway fails
        Pool(16, 4, budget_pages=0)
    assert refused.value.code == kvx.ENOMEM
    with pytest.raises(kvx.KvxError) as too_long:     # longer than the pool
        Pool(16, 17)
    assert too_long.value.code == kvx.EINVAL


def test_id_exhaustion_is_an_error():
    pool = Pool(8, 8)
    assert pool.acquire(9)[0] == -2


def test_failed_growth_keeps_its_extents_for_the_retry():
    # the reference refuses one named extent; a budget of two extents refuses the third
    pool = Pool(16, 0, budget_pages=8)
    rc, _ = pool.acquire(9)
    s = pool.snap()
    assert rc == -1 and s.extent_releases == 0 and s.pages_allocated == 8
    assert s.reclaimable_bytes == 2 * pool.extent_bytes and s.pages_free == 8 and s.pages_active == 0
    assert s.pages_prefix == 0 and s.extent_allocations == 2
    pool.budget(None)
    rc, pages = pool.acquire(9)
    assert rc == 9 and pool.snap().extent_allocations == 3
    pool.release(pages)
    assert pool.reclaim(False) == 3 * pool.extent_bytes and pool.snap().pages_allocated == 0


def test_pressure_reuses_free_pages_and_denies_growth():
    pool = Pool(8, 4)
    rc, active = pool.acquire(2)
    assert rc == 2
    pool.budget(0)
    rc, reused = pool.acquire(1)
    assert rc == 1 and reused[0] == 2
    assert pool.acquire(2)[0] == -1
    assert pool.active(active[0]) and pool.active(active[1]) and pool.active(reused[0])
    assert pool.snap().pages_active == 3
    pool.release(reused)
    pool.release(active)
    assert pool.reclaim(False) == pool.extent_bytes and pool.snap().pages_allocated == 0


def test_pass_releases_every_empty_extent():
    extents = 200
    pool = Pool(4 * extents, 4 * extents)
    rc, pages = pool.acquire(4 * extents)
    assert rc == 4 * extents and pool.snap().pages_allocated == 4 * extents
    pool.release(pages)
    assert pool.snap().reclaimable_bytes == extents * pool.extent_bytes
    before = pool.snap().extent_releases
    assert pool.reclaim(True) == (extents - 1) * pool.extent_bytes
    s = pool.snap()
    assert s.extent_releases == before + extents - 1 and s.reclaimable_bytes == pool.extent_bytes
    assert pool.reclaim(False) == pool.extent_bytes
    assert pool.snap().pages_allocated == 0 and pool.snap().extent_releases == extents


def test_fullest_extent_fills_first_so_cold_extents_drain():
    pool = Pool(12, 12)
    rc, _ = pool.acquire(12)
    assert rc == 12
    pool.release([0, 1, 2, 5, 8, 9])
    assert pool.snap().pages_free == 6 and pool.snap().reclaimable_bytes == 0
    rc, refill = pool.acquire(2)
    assert rc == 2 and refill[0] == 5 and refill[1] in (8, 9)
    rc, again = pool.acquire(1)
    assert rc == 1 and again[0] // 4 == 2
    pool.release([3])
    assert pool.snap().reclaimable_bytes == pool.extent_bytes
    assert pool.reclaim(False) == pool.extent_bytes and pool.snap().pages_allocated == 8


def test_prefix_and_active_references_hold_the_extent():
    pool = Pool(8, 4)
    rc, active = pool.acquire(1)
    assert pool.retain(active[0], True) == 0
    pool.release(active, False)
    assert pool.reclaim(False) == 0 and pool.snap().pages_prefix == 1
    pool.release(active, True)
    assert pool.reclaim(False) == pool.extent_bytes


def test_cache_owns_a_page_once():
    pool = Pool(4, 4)
    rc, active = pool.acquire(1)
    page = active[0]
    assert pool.retain(page, True) == 0 and pool.snap().pages_prefix == 1
    assert pool.retain(page, True) == -1
    pool.release([page], True)
    with pytest.raises(kvx.KvxError):
        pool.release([page], True)
    assert pool.snap().pages_prefix == 0 and pool.active(page)
    pool.release([page])


def test_compaction_empties_the_extent_with_the_fewest_pages():
    pool = held(12, [0, 1, 2, 7, 10, 11])
    assert pool.retain(3, True) == 0
    moves = pool.compact()
    assert moves and moves["first"] == 0 and len(moves["dest"]) == 4 and moves["moved"] == 1
    assert follow(moves, 3) == 7 and follow(moves, 0) == 0 and follow(moves, 8) == 8
    assert not pool.active(3) and pool.active(7)
    s = pool.snap()
    assert (s.pages_active, s.pages_prefix, s.pages_free, s.pages_allocated) == (6, 1, 6, 12)
    assert s.reclaimable_bytes == pool.extent_bytes and s.extent_compactions == 1 and s.pages_moved == 1
    pool.release([7], True)
    pool.release([7], False)
    assert not pool.active(7) and pool.snap().pages_prefix == 0
    assert pool.reclaim(False) == pool.extent_bytes and pool.snap().pages_allocated == 8


def test_compaction_fills_the_fullest_extents_first():
    pool = held(16, [3, 7, 10, 11, 14, 15])
    moves = pool.compact()
    assert moves["first"] == 8 and follow(moves, 8) == 3 and follow(moves, 9) == 7
    assert pool.compact() is None and pool.snap().extent_compactions == 1
    assert pool.snap().pages_moved == 2


def test_compaction_needs_free_pages_in_extents_in_use():
    pool = held(12, [1, 2, 3, 4, 5, 6, 7])
    assert pool.compact() is None
    assert pool.snap().reclaimable_bytes == pool.extent_bytes and pool.snap().extent_compactions == 0
    tight = held(8, [2, 3, 7])
    assert tight.compact() is None


def test_compaction_leaves_fixed_pages_in_place():
    pool = held(16, [3, 7, 10, 11, 14, 15])
    assert pool.compact([0, 4, 9, 13]) is None
    moves = pool.compact([9])
    assert moves["first"] == 12 and follow(moves, 12) == 3 and follow(moves, 13) == 7
    assert follow(moves, 9) == 9 and pool.active(9)
