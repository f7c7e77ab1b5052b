"""GPU parity of quantize-on-append, page copy and path compaction: bit-exact
against the oracle on the same seeded inputs, through the C ABI."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import kvoracle as ko
from richengine_amd import kvx
import kvtestlib as T
import gpulib as Gp

pytestmark = pytest.mark.gpu
H, D = 4, 256
FORMATS = [ko.INT4, ko.INT8, ko.FP8, ko.BF16]


def random_rows(rng, tokens, outliers=True):
    k = rng.standard_normal((H, tokens, D)).astype(np.float32)
    v = rng.standard_normal((H, tokens, D)).astype(np.float32)
    if outliers:
        k[:, :, [3, 77, 130, 255]] *= 20
        v[:, :, [9, 100]] *= 20
    if tokens > 2:
        k[1, 1, :] = 0
        v[2, 0, :] = 0
    return k, v


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("committed,tokens", [(0, 1), (0, 32), (33, 7), (129, 8), (31, 70),
                                              (1000, 257), (0, 2048)])
def test_prefill_store_is_bit_exact(fmt, committed, tokens):
    rng = np.random.default_rng(committed * 7 + tokens + fmt)
    n_pages = (committed + tokens + 31) // 32
    tw = Gp.Twin(fmt, H, D, 2, n_pages)
    pages = tw.pages(n_pages, committed + tokens)
    th, td = tw.tables(pages)
    k, v = random_rows(rng, tokens)
    stride = (tokens + 31) // 32 * 32
    ck, cv = T.chunk_buffers(k, v, stride)
    p = ko.ChunkParams(committed, tokens, stride, n_pages, tw.host.layer(1))
    assert ko.store_chunk(fmt, H, D, ck, cv, th, p) == 1
    kvx.append(tw.dev, 1, Gp.dev(ck), Gp.dev(cv), [td],
               [kvx.ChunkParams(committed, tokens, stride, n_pages)], H * stride * D)
    torch.cuda.synchronize()
    tw.assert_same_bytes()
    tw.close()


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.FP8])
def test_extreme_magnitudes_are_bit_exact(fmt):
    # tiny, huge and subnormal-range rows exercise the fp32 division and the
    # e4m3 subnormal / saturation branches
    rng = np.random.default_rng(fmt)
    tokens = 64
    k, v = random_rows(rng, tokens, outliers=False)
    scales = np.exp(rng.uniform(-60, 60, (H, tokens, 1))).astype(np.float32)
    k, v = k * scales, v * scales[::-1]
    k[0, 5] = np.float32(3.0e38)
    v[3, 7, 3] = np.float32(-3.3e38)
    tw = Gp.Twin(fmt, H, D, 1, 2)
    pages = tw.pages(2, 1)
    th, td = tw.tables(pages)
    ck, cv = T.chunk_buffers(k, v, 64)
    p = ko.ChunkParams(0, tokens, 64, 2, tw.host.layer(0))
    assert ko.store_chunk(fmt, H, D, ck, cv, th, p) == 1
    kvx.append(tw.dev, 0, Gp.dev(ck), Gp.dev(cv), [td], [kvx.ChunkParams(0, tokens, 64, 2)],
               H * 64 * D)
    torch.cuda.synchronize()
    tw.assert_same_bytes()
    tw.close()


def test_bf16_store_keeps_every_bit_pattern():
    bits = np.array([0, 0x8000, 1, 0x8001, 0x007f, 0x0080, 0x4960, 0x7f7f, 0xff7f, 0x7f80, 0xff80,
                     0x7fc3], dtype=np.uint16)
    stride, rows, committed = 64, 33, 31
    ck = bits[np.arange(H * stride * D) % 12].reshape(H, stride, D)
    cv = bits[(np.arange(H * D * stride) + 5) % 12].reshape(H, D, stride)
    tw = Gp.Twin(ko.BF16, H, D, 2, 2)
    pages = tw.pages(2, 3)
    th, td = tw.tables(pages)
    p = ko.ChunkParams(committed, rows, stride, 2, tw.host.layer(1))
    assert ko.store_chunk(ko.BF16, H, D, ck, cv, th, p) == 1
    kvx.append(tw.dev, 1, Gp.dev(ck), Gp.dev(cv), [td], [kvx.ChunkParams(committed, rows, stride, 2)],
               H * stride * D)
    torch.cuda.synchronize()
    tw.assert_same_bytes()
    tw.close()


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16])
@pytest.mark.parametrize("lanes,rows,max_rows", [(3, 8, 15), (4, 15, 15), (40, 1, 15), (4, 16, 16)])
def test_verify_store_lanes(fmt, lanes, rows, max_rows):
    rng = np.random.default_rng(lanes * 100 + rows)
    committed = [int(x) for x in rng.integers(0, 1500, lanes)]
    committed[0] = 0
    counts = [(c + rows + 31) // 32 for c in committed]
    tw = Gp.Twin(fmt, H, D, 2, sum(counts))
    ids = tw.pages(sum(counts), 11)
    host_tables, dev_tables, first = [], [], 0
    for n in counts:
        th, td = tw.tables(ids[first:first + n])
        host_tables.append(th)
        dev_tables.append(td)
        first += n
    ck = ko.f32_to_bf16(rng.standard_normal((lanes, H, 32, D)).astype(np.float32)).reshape(lanes, H, 32, D)
    cv = ko.f32_to_bf16(rng.standard_normal((lanes, H, D, 32)).astype(np.float32)).reshape(lanes, H, D, 32)
    hp = [ko.ChunkParams(committed[i], rows, 32, counts[i], tw.host.layer(1)) for i in range(lanes)]
    assert ko.store_verify(fmt, H, D, ck, cv, host_tables, hp, max_rows) == lanes
    dp = [kvx.ChunkParams(committed[i], rows, 32, counts[i]) for i in range(lanes)]
    kvx.append(tw.dev, 1, Gp.dev(ck), Gp.dev(cv), dev_tables, dp, H * 32 * D, verify_max_rows=max_rows)
    torch.cuda.synchronize()
    tw.assert_same_bytes()
    tw.close()


def test_invalid_parameters_enqueue_nothing():
    tw = Gp.Twin(ko.INT8, H, D, 1, 4)
    pages = tw.pages(4, 2)
    th, td = tw.tables(pages)
    poison = np.full(tw.dev.extent_bytes, 0xA5, dtype=np.uint8)
    for e in range(tw.extents):
        tw.dev.extent_write(e, poison)
    ck = Gp.dev(np.full((H, 32, D), 0x3F80, dtype=np.uint16))
    bad = [kvx.ChunkParams(40, 0, 32, 4), kvx.ChunkParams(40, 8, 24, 4), kvx.ChunkParams(40, 8, 32, 1),
           kvx.ChunkParams(262159 - 3, 8, 32, 9000), kvx.ChunkParams(0, 2049, 2080, 99)]
    for p in bad:
        with pytest.raises(kvx.KvxError) as err:
            kvx.append(tw.dev, 0, ck, ck, [td], [p], H * 32 * D)
        assert err.value.code == kvx.EINVAL
    with pytest.raises(kvx.KvxError):
        kvx.append(tw.dev, 0, ck, ck, [td], [kvx.ChunkParams(40, 16, 32, 4)], H * 32 * D,
                   verify_max_rows=15)
    with pytest.raises(kvx.KvxError) as err:
        kvx.append(tw.dev, 7, ck, ck, [td], [kvx.ChunkParams(40, 8, 32, 4)], H * 32 * D)
    assert err.value.code == kvx.ERANGE
    torch.cuda.synchronize()
    for e in range(tw.extents):
        assert (tw.dev.extent_read(e) == 0xA5).all()
    tw.close()


def fill_twin(tw, total, seed, layers=(0, 1)):
    n_pages = (total + 31) // 32
    pages = tw.pages(n_pages, seed)
    th, td = tw.tables(pages)
    rng = np.random.default_rng(seed)
    k, v = random_rows(rng, total)
    stride = (total + 31) // 32 * 32
    ck, cv = T.chunk_buffers(k, v, stride)
    for layer in layers:
        p = ko.ChunkParams(0, total, stride, n_pages, tw.host.layer(layer))
        assert ko.store_chunk(tw.fmt, H, D, ck, cv, th, p) == 1
    tw.upload()
    return pages, th, td


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("committed,path", [(0, [0, 2, 5]), (27, [0, 1, 4, 9, 15]), (61, [0, 3]),
                                              (100, [0, 1, 2, 3]), (31, [0, 15]),
                                              (5, list(range(0, 16, 2)))])
def test_path_compaction_is_bit_exact(fmt, committed, path):
    rows = 16
    tw = Gp.Twin(fmt, H, D, 2, (committed + rows + 31) // 32)
    pages, th, td = fill_twin(tw, committed + rows, seed=committed + len(path))
    rp = np.zeros((1, 16), dtype=np.uint32)
    rp[0, :len(path)] = path
    count = np.array([len(path)], dtype=np.uint32)
    hp = ko.ChunkParams(committed, rows, 32, len(pages), tw.host.layer(1))
    ko.compact_tree(fmt, H, D, [th], [hp], rp, count, 16)
    kvx.compact_path(tw.dev, 1, [td], [kvx.ChunkParams(committed, rows, 32, len(pages))],
                     Gp.dev(rp), Gp.dev(count), 16)
    torch.cuda.synchronize()
    tw.assert_same_bytes()
    tw.close()


def test_compaction_of_every_layer_and_many_lanes():
    fmt, lanes, rows = ko.INT4, 5, 16
    rng = np.random.default_rng(77)
    committed = [int(x) for x in rng.integers(0, 300, lanes)]
    counts = [(c + rows + 31) // 32 for c in committed]
    tw = Gp.Twin(fmt, H, D, 3, sum(counts))
    ids = tw.pages(sum(counts), 5)
    hts, dts, first = [], [], 0
    for lane, n in enumerate(counts):
        th, td = tw.tables(ids[first:first + n])
        hts.append(th)
        dts.append(td)
        first += n
        total = committed[lane] + rows
        k, v = random_rows(rng, total)
        stride = (total + 31) // 32 * 32
        ck, cv = T.chunk_buffers(k, v, stride)
        for layer in range(3):
            p = ko.ChunkParams(0, total, stride, n, tw.host.layer(layer))
            assert ko.store_chunk(fmt, H, D, ck, cv, th, p) == 1
    tw.upload()
    rp = np.zeros((lanes, 16), dtype=np.uint32)
    count = np.zeros(lanes, dtype=np.uint32)
    for lane in range(lanes):
        n = int(rng.integers(0, 9))
        path = np.sort(rng.choice(np.arange(1, 16), size=max(n - 1, 0), replace=False))
        if n:
            rp[lane, 0] = 0
            rp[lane, 1:n] = path
        count[lane] = n
    for layer in range(3):
        hp = [ko.ChunkParams(committed[i], rows, 32, counts[i], tw.host.layer(layer)) for i in range(lanes)]
        ko.compact_tree(fmt, H, D, hts, hp, rp, count, 16)
    dp = [kvx.ChunkParams(committed[i], rows, 32, counts[i]) for i in range(lanes)]
    kvx.compact_path(tw.dev, kvx.ALL_LAYERS, dts, dp, Gp.dev(rp), Gp.dev(count), 16)
    torch.cuda.synchronize()
    tw.assert_same_bytes()
    tw.close()


def test_malformed_path_moves_nothing():
    tw = Gp.Twin(ko.INT8, H, D, 1, 2)
    pages, th, td = fill_twin(tw, 48, seed=1, layers=(0,))
    before = [tw.dev.extent_read(e) for e in range(tw.extents)]
    dp = [kvx.ChunkParams(20, 16, 32, 2)]
    for path, n in (([0, 5, 3], 3), ([0, 16], 2), ([2, 1], 2), ([0] * 16, 16)):
        rp = np.zeros((1, 16), dtype=np.uint32)
        rp[0, :len(path)] = path
        kvx.compact_path(tw.dev, 0, [td], dp, Gp.dev(rp), Gp.dev(np.array([n], dtype=np.uint32)), 16)
    kvx.compact_path(tw.dev, 0, [td], dp, Gp.dev(np.zeros((1, 16), dtype=np.uint32)),
                     Gp.dev(np.array([17], dtype=np.uint32)), 16)
    torch.cuda.synchronize()
    for e in range(tw.extents):
        assert np.array_equal(tw.dev.extent_read(e), before[e])
    tw.close()


@pytest.mark.parametrize("fmt", FORMATS)
def test_page_copy_is_bit_exact(fmt):
    tw = Gp.Twin(fmt, H, D, 3, 6)
    pages, th, td = fill_twin(tw, 96, seed=fmt, layers=(0, 1, 2))
    used = set(int(p) for p in pages)
    free = [p for p in range(tw.dev.page_count) if p not in used]
    copies = [(int(pages[0]), free[0]), (int(pages[2]), free[1])]
    assert tw.host.copy_pages(copies) == 0
    tw.dev.copy_pages(copies)
    torch.cuda.synchronize()
    tw.assert_same_bytes()
    assert np.array_equal(tw.dev.page_read(free[0]), tw.host.page_read(int(pages[0])))
    # chains and shared destinations are refused, and refused batches copy nothing
    for bad in ([(int(pages[0]), free[2]), (free[2], free[3])], [(int(pages[0]), free[2]), (int(pages[1]), free[2])]):
        with pytest.raises(kvx.KvxError) as err:
            tw.dev.copy_pages(bad)
        assert err.value.code == kvx.EINVAL
    tw.dev.release(tw.extents - 1)
    victim = (tw.extents - 1) * tw.extent_pages
    ok_src = [p for p in used if p // tw.extent_pages != tw.extents - 1][0]
    dst = [p for p in free if p // tw.extent_pages != tw.extents - 1][-1]
    before = tw.dev.page_read(dst)
    with pytest.raises(kvx.KvxError) as err:
        tw.dev.copy_pages([(ok_src, dst), (ok_src, victim)])
    assert err.value.code == kvx.ESTATE
    with pytest.raises(kvx.KvxError) as err:
        tw.dev.copy_pages([(ok_src, tw.dev.page_count)])
    assert err.value.code == kvx.ERANGE
    assert np.array_equal(tw.dev.page_read(dst), before)
    tw.close()


def test_pool_compaction_moves_page_bytes_on_the_device():
    # elastic_kv_pool_test.cpp:261-293 on real extents: page 3 moves to page 7
    st = kvx.Storage(2, H, D, ko.INT4, 12, 4)
    pool = kvx.Pool(st, 12)
    assert pool.acquire(12) == list(range(12))
    rng = np.random.default_rng(0)
    content = {p: rng.integers(0, 256, st.bytes_per_page, dtype=np.uint8) for p in range(12)}
    for p, data in content.items():
        st.page_write(p, data)
    for p in (0, 1, 2, 7, 10, 11):
        pool.release(p)
    pool.retain(3, prefix_owner=True)
    moves = pool.compact_extent()
    torch.cuda.synchronize()
    assert moves["first"] == 0 and moves["dest"] == [0, 1, 2, 7] and moves["moved"] == 1
    assert np.array_equal(st.page_read(7), content[3])
    assert not pool.page_active(3) and pool.page_active(7)
    s = pool.snapshot()
    assert (s.pages_active, s.pages_prefix, s.pages_free, s.pages_allocated) == (6, 1, 6, 12)
    assert s.extent_compactions == 1 and s.pages_moved == 1
    assert pool.reclaim_empty(False) == st.extent_bytes
    assert pool.snapshot().pages_allocated == 8
    with pytest.raises(kvx.KvxError):
        st.entries_host([0])  # the released extent's pages have no entries
    pool.close()
    st.close()


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("pinned", [False, True])
def test_page_export_and_import_are_the_wire_bytes(fmt, pinned):
    """kv_page_export writes exactly the bytes PageStorage::spans lists for each page
    (the oracle's page_read, pinned by its own tests), into device memory or pinned host
    memory; kv_import puts them back into other pages byte for byte; invalid lists
    enqueue nothing."""
    rng = np.random.default_rng(70 + fmt)
    tokens, layers = 200 * 32, 3          # 200 pages: more than one launch of 128
    n_pages = tokens // 32
    tw = Gp.Twin(fmt, H, D, layers, 2 * n_pages + 4)
    pages = tw.pages(2 * n_pages, 71)
    source, target = pages[:n_pages], pages[n_pages:]
    _, td = tw.tables(source)
    for layer in range(layers):
        for done in range(0, tokens, 1600):
            k, v = random_rows(rng, 1600)
            ck, cv = T.chunk_buffers(k, v, 1600)
            kvx.append(tw.dev, layer, Gp.dev(ck), Gp.dev(cv), [td],
                       [kvx.ChunkParams(done, 1600, 1600, n_pages)], H * 1600 * D)
    torch.cuda.synchronize()
    tw.download()
    page_bytes = tw.dev.bytes_per_page
    want = np.concatenate([tw.host.page_read(int(p)) for p in source])
    buffer = torch.zeros(n_pages * page_bytes, dtype=torch.uint8, pin_memory=pinned,
                         device="cpu" if pinned else "cuda")
    tw.dev.export_pages(source, buffer)
    torch.cuda.synchronize()
    assert np.array_equal(buffer.cpu().numpy(), want)
    before = [tw.dev.page_read(int(p)) for p in source[::37]]
    tw.dev.import_pages(target, buffer)
    torch.cuda.synchronize()
    for a, b in list(zip(source, target))[::17]:
        assert np.array_equal(tw.dev.page_read(int(b)), tw.host.page_read(int(a)))
    assert all(np.array_equal(x, tw.dev.page_read(int(p))) for x, p in zip(before, source[::37]))
    # an invalid page, an unallocated extent's page or a repeated destination: nothing enqueued
    probe = tw.dev.page_read(int(target[0]))
    for bad in ([int(target[0]), tw.dev.page_count], [int(target[0]), int(target[0])]):
        with pytest.raises(kvx.KvxError):
            tw.dev.import_pages(bad, buffer)
    with pytest.raises(kvx.KvxError):
        tw.dev.export_pages([tw.dev.page_count + 5], buffer)
    torch.cuda.synchronize()
    assert np.array_equal(probe, tw.dev.page_read(int(target[0])))
    tw.close()
