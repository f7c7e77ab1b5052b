"""Oracle tree-path compaction and whole-page copy.

The reference holds no test of the compaction kernel
(decode/paged_attention_store.metal:198-278), so it is pinned here by an
independent gather-all-then-scatter in numpy -- equivalent to the forward
copy because a strictly increasing path has path[i] >= i.  Page copy follows
dev/tests/engine/q8_page_storage_test.mm:251-260 (a refused batch copies
nothing) and PageStorage.mm:95-114.
"""
import numpy as np
import pytest

from oracle import kvoracle as ko
import kvtestlib as T

H, D = 4, 256


def appended(fmt, committed, rows, seed):
    total = committed + rows
    n_pages = (total + 31) // 32
    store = T.make_store(fmt, H, D, 2, n_pages)
    pages = T.mixed_pages(store.extent_pages, store.page_count // store.extent_pages, n_pages, seed)
    table = store.entries(pages)
    rng = np.random.default_rng(seed)
    k = rng.standard_normal((H, total, D)).astype(np.float32)
    v = rng.standard_normal((H, total, D)).astype(np.float32)
    stride = (total + 31) // 32 * 32
    ck, cv = T.chunk_buffers(k, v, stride)
    for layer in (0, 1):
        p = ko.ChunkParams(0, total, stride, n_pages, store.layer(layer))
        assert ko.store_chunk(fmt, H, D, ck, cv, table, p) == 1
    return store, pages, table


def token_rows(store, pages, layer, token):
    """Everything one token holds in one layer, as comparable arrays."""
    kc, ks, vc, vs = T.page_codes(store, layer, int(pages[token // 32]))
    s = token % 32
    return kc[:, s].copy(), ks[:, s].copy(), vc[:, s].copy(), vs[:, s].copy()


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16, ko.FP8])
@pytest.mark.parametrize("committed,path", [(0, [0, 2, 5]), (27, [0, 1, 4, 9, 15]), (61, [0, 3]),
                                              (100, [0, 1, 2, 3]), (31, [0, 15])])
def test_compaction_matches_gather_then_scatter(fmt, committed, path):
    rows = 16
    store, pages, table = appended(fmt, committed, rows, seed=committed + len(path))
    before = {(layer, t): token_rows(store, pages, layer, t)
              for layer in (0, 1) for t in range(committed + rows)}
    snapshot = [store.extent(e).copy() for e in range(store.page_count // store.extent_pages)]
    rp = np.zeros((1, 16), dtype=np.uint32)
    rp[0, :len(path)] = path
    count = np.array([len(path)], dtype=np.uint32)
    p = ko.ChunkParams(committed, rows, 32, len(pages), store.layer(1))
    ko.compact_tree(fmt, H, D, [table], [p], rp, count, 16)
    for t in range(committed + rows):
        i = t - committed
        src = committed + path[i] if 0 <= i < len(path) else t
        for got, want in zip(token_rows(store, pages, 1, t), before[(1, src)]):
            assert np.array_equal(got, want, equal_nan=True)
        for got, want in zip(token_rows(store, pages, 0, t), before[(0, t)]):
            assert np.array_equal(got, want, equal_nan=True)  # other layers untouched
    # only the moved tokens' bytes changed anywhere in the pool
    changed = sum(int((store.extent(e) != snapshot[e]).sum())
                  for e in range(store.page_count // store.extent_pages))
    per_token = {ko.INT4: 2 * 128 + 8, ko.INT8: 2 * 256 + 8, ko.FP8: 2 * 256 + 8, ko.BF16: 1024}[fmt] * H
    moved = sum(1 for i, s in enumerate(path) if s != i)
    assert changed <= moved * per_token


def test_identity_path_and_zero_count_move_nothing():
    store, pages, table = appended(ko.INT4, 40, 16, seed=3)
    snapshot = [store.extent(e).copy() for e in range(store.page_count // store.extent_pages)]
    p = ko.ChunkParams(40, 16, 32, len(pages), store.layer(1))
    rp = np.arange(16, dtype=np.uint32).reshape(1, 16)
    assert ko.compact_tree(ko.INT4, H, D, [table], [p], rp, np.array([8], dtype=np.uint32), 16) == 0
    assert ko.compact_tree(ko.INT4, H, D, [table], [p], rp[:, ::-1].copy(),
                           np.array([0], dtype=np.uint32), 16) == 0
    for e, snap in enumerate(snapshot):
        assert np.array_equal(store.extent(e), snap)


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16])
def test_page_copy_moves_every_tensor_of_every_layer(fmt):
    store, pages, table = appended(fmt, 0, 96, seed=12)
    free = [p for p in range(store.page_count) if p not in set(int(x) for x in pages)]
    src, dst = int(pages[1]), free[0]
    want = store.page_read(src)
    assert want.any() and not store.page_read(dst).any()
    others = {int(p): store.page_read(int(p)) for p in pages}
    assert store.copy_pages([(src, dst)]) == 0
    assert np.array_equal(store.page_read(dst), want)
    for p, data in others.items():
        assert np.array_equal(store.page_read(p), data)  # source and neighbours untouched
    assert want.size == store.bytes_per_page


def test_refused_copy_batch_copies_nothing():
    store, pages, table = appended(ko.INT8, 0, 64, seed=13)
    n_ext = store.page_count // store.extent_pages
    assert store.release(n_ext - 1) == 0
    victim = (n_ext - 1) * store.extent_pages
    ok_pages = [int(p) for p in pages if int(p) // store.extent_pages != n_ext - 1]
    free = [p for p in range(victim) if p not in set(ok_pages)]
    before = store.page_read(free[0]).copy()
    assert store.copy_pages([(ok_pages[0], free[0]), (ok_pages[0], victim)]) == -1
    assert np.array_equal(store.page_read(free[0]), before)
    assert store.allocate(n_ext - 1) == 0 and store.allocate(n_ext - 1) == -1
