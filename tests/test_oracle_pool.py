"""Oracle page pool: the reference's fifteen pool cases with their exact page
ids and moves (dev/tests/engine/elastic_kv_pool_test.cpp:40-383), restated
against the oracle's pool."""
import ctypes as C

import numpy as np
import pytest

from oracle import kvoracle as ko

L = ko.lib()
EXTENT_BYTES = 4 * 100
NO_LIMIT = 0xFFFFFFFF


class Pool:
    def __init__(self, pages, runway, extent_pages=4, budget=NO_LIMIT, blocked=False, refused=-1):
        self.extent_pages = extent_pages
        self.n = pages
        # a blocked storage refuses the runway too
        self.h = None
        if blocked:
            probe = L.ko_pool_create(pages, 100, extent_pages, 0, budget)
            L.ko_pool_set_growth_blocked(probe, 1)
            self.h = probe
            return
        self.h = L.ko_pool_create(pages, 100, extent_pages, runway, budget)
        if self.h and refused >= 0:
            L.ko_pool_set_refused_extent(self.h, refused)

    def acquire(self, count):
        out = np.zeros(max(count, 1), dtype=np.uint32)
        rc = L.ko_pool_acquire(self.h, count, ko.ptr(out))
        return rc, list(out[:count]) if rc == count else []

    def release(self, pages, prefix=False):
        for p in pages:
            assert L.ko_pool_release(self.h, int(p), int(prefix)) == 0

    def retain(self, page, prefix):
        return L.ko_pool_retain(self.h, page, int(prefix))

    def snap(self):
        s = ko.PoolSnapshot()
        L.ko_pool_snapshot_get(self.h, C.byref(s))
        return s

    def reclaim(self, keep, limit=NO_LIMIT):
        return L.ko_pool_reclaim_empty(self.h, int(keep), limit)

    def active(self, page):
        return bool(L.ko_pool_page_active(self.h, page))

    def compact(self, fixed=()):
        fixed = np.array(list(fixed), dtype=np.uint32)
        first = C.c_uint32()
        dest = np.zeros(self.extent_pages, dtype=np.uint32)
        copies = (ko.PageCopy * self.extent_pages)()
        n = C.c_uint32()
        rc = L.ko_pool_compact_extent(self.h, ko.ptr(fixed) if len(fixed) else None, len(fixed),
                                      C.byref(first), ko.ptr(dest), copies, C.byref(n))
        if rc == 0:
            return None
        return dict(first=first.value, dest=list(dest), copies=[(c.from_, c.to) for c in copies[:n.value]])

    def content(self, page):
        return L.ko_pool_content(self.h, page)


def follow(moves, page):
    if moves and moves["first"] <= page < moves["first"] + len(moves["dest"]):
        return moves["dest"][page - moves["first"]]
    return page


def held(pages, released):
    pool = Pool(pages, pages)
    for p in range(pages):
        L.ko_pool_set_content(pool.h, p, 100 + p)
    rc, got = pool.acquire(pages)
    assert rc == pages
    pool.release(released)
    return pool


def test_growth_packs_allocated_extents():
    pool = Pool(12, 4)
    rc, pages = pool.acquire(5)
    assert rc == 5 and pages[0] == 0 and pages[3] == 3 and pages[4] == 4
    s = pool.snap()
    assert (s.pages_allocated, s.pages_active, s.pages_free, s.allocated_bytes) == (8, 5, 3, 800)
    pool.release(pages)
    assert pool.reclaim(True) == EXTENT_BYTES
    s = pool.snap()
    assert s.pages_allocated == 4 and s.reclaimable_bytes == EXTENT_BYTES
    assert s.extent_allocations == 2 and s.extent_releases == 1


def test_runway_is_allocated_through_the_pool():
    pool = Pool(16, 6)
    s = pool.snap()
    assert s.extent_allocations == 2 and s.pages_allocated == 8 and s.reclaimable_bytes == 2 * EXTENT_BYTES
    assert L.ko_pool_extent_allocated(pool.h, 0) and L.ko_pool_extent_allocated(pool.h, 1)
    assert not L.ko_pool_extent_allocated(pool.h, 2)
    assert pool.reclaim(True) == EXTENT_BYTES
    s = pool.snap()
    assert s.extent_allocations - s.extent_releases == 1 and s.pages_allocated == 4
    assert L.ko_pool_create(16, 100, 4, 4, 0) is None       # a refused runway fails
    assert L.ko_pool_create(16, 100, 4, 17, NO_LIMIT) is None  # longer than the pool


def test_id_exhaustion_is_an_error():
    pool = Pool(8, 8)
    assert pool.acquire(9)[0] == -2


def test_failed_growth_keeps_its_extents_for_the_retry():
    pool = Pool(16, 0, refused=2)
    rc, _ = pool.acquire(9)
    s = pool.snap()
    assert rc == -1 and s.extent_releases == 0 and s.pages_allocated == 8
    assert s.reclaimable_bytes == 2 * EXTENT_BYTES and s.pages_free == 8 and s.pages_active == 0
    assert s.pages_prefix == 0 and s.extent_allocations == 2
    L.ko_pool_set_refused_extent(pool.h, -1)
    rc, pages = pool.acquire(9)
    assert rc == 9 and pool.snap().extent_allocations == 3
    pool.release(pages)
    assert pool.reclaim(False) == 3 * EXTENT_BYTES and pool.snap().pages_allocated == 0


def test_pressure_reuses_free_pages_and_denies_growth():
    pool = Pool(8, 4)
    rc, active = pool.acquire(2)
    assert rc == 2
    L.ko_pool_set_growth_blocked(pool.h, 1)
    rc, reused = pool.acquire(1)
    assert rc == 1 and reused[0] == 2
    assert pool.acquire(2)[0] == -1
    assert pool.active(active[0]) and pool.active(active[1]) and pool.active(reused[0])
    assert pool.snap().pages_active == 3
    pool.release(reused)
    pool.release(active)
    assert pool.reclaim(False) == EXTENT_BYTES and pool.snap().pages_allocated == 0


def test_pass_releases_every_empty_extent():
    extents = 200
    pool = Pool(4 * extents, 4 * extents)
    rc, pages = pool.acquire(4 * extents)
    assert rc == 4 * extents and pool.snap().pages_allocated == 4 * extents
    pool.release(pages)
    assert pool.snap().reclaimable_bytes == extents * EXTENT_BYTES
    before = pool.snap().extent_releases
    assert pool.reclaim(True) == (extents - 1) * EXTENT_BYTES
    s = pool.snap()
    assert s.extent_releases == before + extents - 1 and s.reclaimable_bytes == EXTENT_BYTES
    assert pool.reclaim(False) == EXTENT_BYTES
    assert pool.snap().pages_allocated == 0 and pool.snap().extent_releases == extents


def test_fullest_extent_fills_first_so_cold_extents_drain():
    pool = Pool(12, 12)
    rc, all_pages = pool.acquire(12)
    assert rc == 12
    pool.release([0, 1, 2, 5, 8, 9])
    assert pool.snap().pages_free == 6 and pool.snap().reclaimable_bytes == 0
    rc, refill = pool.acquire(2)
    assert rc == 2 and refill[0] == 5 and refill[1] in (8, 9)
    rc, again = pool.acquire(1)
    assert rc == 1 and again[0] // 4 == 2
    pool.release([3])
    assert pool.snap().reclaimable_bytes == EXTENT_BYTES
    assert pool.reclaim(False) == EXTENT_BYTES and pool.snap().pages_allocated == 8


def test_prefix_and_active_references_hold_the_extent():
    pool = Pool(8, 4)
    rc, active = pool.acquire(1)
    assert pool.retain(active[0], True) == 0
    pool.release(active, False)
    assert pool.reclaim(False) == 0 and pool.snap().pages_prefix == 1
    pool.release(active, True)
    assert pool.reclaim(False) == EXTENT_BYTES


def test_cache_owns_a_page_once():
    pool = Pool(4, 4)
    rc, active = pool.acquire(1)
    page = active[0]
    assert pool.retain(page, True) == 0 and pool.snap().pages_prefix == 1
    assert pool.retain(page, True) == -1
    assert L.ko_pool_release(pool.h, page, 1) == 0
    assert L.ko_pool_release(pool.h, page, 1) == -1
    assert pool.snap().pages_prefix == 0 and pool.active(page)
    pool.release([page])


def test_compaction_empties_the_extent_with_the_fewest_pages():
    pool = held(12, [0, 1, 2, 7, 10, 11])
    assert pool.retain(3, True) == 0
    moves = pool.compact()
    assert moves and moves["first"] == 0 and len(moves["dest"]) == 4
    assert follow(moves, 3) == 7 and follow(moves, 0) == 0 and follow(moves, 8) == 8
    assert moves["copies"] == [(3, 7)] and pool.content(7) == 103
    assert not pool.active(3) and pool.active(7)
    s = pool.snap()
    assert (s.pages_active, s.pages_prefix, s.pages_free, s.pages_allocated) == (6, 1, 6, 12)
    assert s.reclaimable_bytes == EXTENT_BYTES and s.extent_compactions == 1 and s.pages_moved == 1
    pool.release([7], True)
    pool.release([7], False)
    assert not pool.active(7) and pool.snap().pages_prefix == 0
    assert pool.reclaim(False) == EXTENT_BYTES and pool.snap().pages_allocated == 8


def test_compaction_fills_the_fullest_extents_first():
    pool = held(16, [3, 7, 10, 11, 14, 15])
    moves = pool.compact()
    assert moves["first"] == 8 and follow(moves, 8) == 3 and follow(moves, 9) == 7
    assert pool.content(3) == 108 and pool.content(7) == 109
    assert pool.compact() is None and pool.snap().extent_compactions == 1
    assert pool.snap().pages_moved == 2


def test_compaction_needs_free_pages_in_extents_in_use():
    pool = held(12, [1, 2, 3, 4, 5, 6, 7])
    assert pool.compact() is None
    assert pool.snap().reclaimable_bytes == EXTENT_BYTES and pool.snap().extent_compactions == 0
    tight = held(8, [2, 3, 7])
    assert tight.compact() is None


def test_compaction_leaves_fixed_pages_in_place():
    pool = held(16, [3, 7, 10, 11, 14, 15])
    assert pool.compact([0, 4, 9, 13]) is None
    moves = pool.compact([9])
    assert moves["first"] == 12 and follow(moves, 12) == 3 and follow(moves, 13) == 7
    assert follow(moves, 9) == 9 and pool.active(9)
