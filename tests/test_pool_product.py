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


def test_random_walk_in_lockstep_with_the_oracle_pool():
    """Page ids, refusals, reclaimed bytes and compaction moves of the product's pool against
    the oracle's restatement of the reference pool over a long random walk: acquisitions of
    random sizes (some refused by a budget that moves), releases in random order, references
    to pages that are free, prefix references, reclaims with and without a runway and a limit,
    compactions with and without fixed pages."""
    import numpy as np
    from oracle import kvoracle as ko
    KO = ko.lib()
    rng = np.random.default_rng(20260)
    for extent_pages, extents in ((4, 6), (5, 9), (16, 5)):
        pages = extent_pages * extents
        runway = int(rng.integers(0, pages + 1))
        mine = Pool(pages, runway, extent_pages)
        theirs = KO.ko_pool_create(pages, mine.page_bytes, extent_pages, runway, NO_LIMIT)
        assert theirs
        held_active, held_prefix = [], []

        def same_books():
            a, b = mine.snap(), ko.PoolSnapshot()
            KO.ko_pool_snapshot_get(theirs, C.byref(b))
            for field in ("pages_allocated", "pages_free", "pages_active", "pages_prefix",
                          "allocated_bytes", "reclaimable_bytes", "extent_allocations",
                          "extent_releases", "extent_compactions", "pages_moved"):
                assert getattr(a, field) == getattr(b, field), field

        for step in range(3000):
            op = rng.integers(0, 100)
            if op < 30:
                count = int(rng.integers(0, extent_pages * 2 + 1))
                out = np.zeros(max(count, 1), dtype=np.uint32)
                rc_theirs = KO.ko_pool_acquire(theirs, count, ko.ptr(out))
                rc_mine, got = mine.acquire(count)
                assert rc_mine == rc_theirs, (step, count)
                if rc_mine == count:
                    assert got == list(out[:count]), (step, got, list(out[:count]))
                    held_active += got
            elif op < 55 and held_active:
                page = held_active.pop(int(rng.integers(0, len(held_active))))
                assert KO.ko_pool_release(theirs, page, 0) == 0
                mine.release([page])
            elif op < 62 and held_prefix:
                page = held_prefix.pop(int(rng.integers(0, len(held_prefix))))
                assert KO.ko_pool_release(theirs, page, 1) == 0
                mine.release([page], True)
            elif op < 72:
                # a reference to any page of the pool: held, free in the middle of a stack,
                # or without memory (refused by both)
                page, prefix = int(rng.integers(0, pages)), bool(rng.integers(0, 2))
                rc_theirs = KO.ko_pool_retain(theirs, page, int(prefix))
                rc_mine = mine.retain(page, prefix)
                assert rc_mine == rc_theirs, (step, page, prefix)
                if rc_mine == 0:
                    (held_prefix if prefix else held_active).append(page)
            elif op < 80:
                keep, limit = bool(rng.integers(0, 2)), int(rng.choice([0, 1, 2, NO_LIMIT]))
                assert mine.reclaim(keep, limit) == KO.ko_pool_reclaim_empty(theirs, int(keep), limit)
            elif op < 84:
                # the budget moves: between nothing and the whole pool
                budget = int(rng.integers(0, extents + 1))
                mine.budget(None if budget == extents else budget * extent_pages)
                KO.ko_pool_set_budget_pages(theirs, NO_LIMIT if budget == extents
                                            else budget * extent_pages)
            else:
                fixed = [int(p) for p in rng.choice(pages, size=int(rng.integers(0, 3)), replace=False)]
                arr = np.array(fixed, dtype=np.uint32)
                first, n = C.c_uint32(), C.c_uint32()
                dest = np.zeros(extent_pages, dtype=np.uint32)
                copies = (ko.PageCopy * extent_pages)()
                moved = KO.ko_pool_compact_extent(theirs, ko.ptr(arr) if fixed else None, len(fixed),
                                                  C.byref(first), ko.ptr(dest), copies, C.byref(n))
                moves = mine.compact(fixed)
                assert (moves is not None) == bool(moved), (step, fixed)
                if moves:
                    assert moves["first"] == first.value and moves["dest"] == list(dest), step
                    assert moves["moved"] == n.value
                    held_active = [follow(moves, p) for p in held_active]
                    held_prefix = [follow(moves, p) for p in held_prefix]
            if step % 50 == 0:
                same_books()
                for page in range(pages):
                    assert mine.active(page) == bool(KO.ko_pool_page_active(theirs, page))
        same_books()
        KO.ko_pool_destroy(theirs)
