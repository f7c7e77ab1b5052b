"""The five benchmark configurations at their full sizes, as parity tests.

Where the scalar oracle finishes in seconds the device result is compared with
it directly (configs 1-3, sampled tiles of 4 and 5); past that, size-independent
properties carry the check: placement invariance (the same bytes behind any
page ids give the same output bits), shared-prefix pages against private
copies, append -> tree verify -> path compaction leaving exactly the oracle's
page bytes.  Histories are written by the device append (pinned bit-exact in
test_gpu_append.py) and copied into the oracle store.
"""
import numpy as np
import pytest
import torch

from oracle import kvoracle as ko
from richengine_amd import kvx
import gpulib as Gp
import kvtestlib as T

pytestmark = pytest.mark.gpu

H, G, D = 4, 6, 256
QH = H * G


def tol(fmt):
    return 1e-2 if fmt == ko.FP8 else 2e-3


def device_history(tw, layer, table_dev, entries, first, count, gen, outliers=False):
    """Appends `count` random tokens at position `first` through kv_append."""
    done = 0
    while done < count:
        n = min(2048, count - done)
        stride = (n + 31) // 32 * 32
        k = torch.randn((H, stride, D), generator=gen, device="cuda")
        v = torch.randn((H, D, stride), generator=gen, device="cuda")
        if outliers:  # a few channels 20x larger, as quantized KV caches see
            k[:, :, [3, 77, 130, 255]] *= 20
            v[:, [5, 64, 131, 250], :] *= 20
        kvx.append(tw.dev, layer, k.bfloat16(), v.bfloat16(), [table_dev],
                   [kvx.ChunkParams(first + done, n, stride, entries)], H * stride * D)
        done += n


def bf16_rows(shape, seed):
    rng = np.random.default_rng(seed)
    return ko.f32_to_bf16(rng.standard_normal(shape).astype(np.float32)).reshape(shape)


def decode_on_device(tw, layer, q, tables, committed, counts, splits):
    lanes = len(committed)
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], splits[i], 1, 1, 0.0)
          for i in range(lanes)]
    out = torch.zeros((lanes, H, 1, G, D), dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH) + 256, dtype=torch.uint8, device="cuda")
    kvx.attend_decode(tw.dev, layer, QH, Gp.dev(q), out, tables, dp, 1, ws)
    torch.cuda.synchronize()
    return Gp.host_u16(out)[:, :, 0]


def decode_on_oracle(tw, layer, q, tables, committed, counts, splits):
    lanes = len(committed)
    want = np.zeros((lanes, H, G, D), dtype=np.uint16)
    want32 = np.zeros((lanes, H, G, D), dtype=np.float32)
    for i in range(lanes):
        q1 = np.zeros((1, H, 32, G, D), dtype=np.uint16)
        q1[0, :, 0] = q[i, :, 0]
        hp = ko.VerifyParams(committed[i], counts[i], tw.host.layer(layer), splits[i], splits[i], 1, 1, 0.0)
        n, o, o32 = ko.attend_verify(tw.fmt, H, G, D, q1, [tables[i]], [hp])
        assert n == 1
        want[i], want32[i] = o[0, :, 0], o32[0, :, 0]
    return want, want32


def test_config1_int8_plumbing():
    # int8, one layer, batch 1: 4096 tokens with outlier channels, one decode step
    tw = Gp.Twin(ko.INT8, H, D, 1, 130)
    pages = tw.pages(129, seed=1)
    th, td = tw.tables(pages)
    rng = np.random.default_rng(1)
    done = 0
    while done < 4097:   # both stores append the same chunks: bytes must agree
        n = min(2048, 4097 - done)
        k = rng.standard_normal((H, n, D)).astype(np.float32)
        v = rng.standard_normal((H, n, D)).astype(np.float32)
        k[:, :, [3, 77, 130, 255]] *= 20
        stride = (n + 31) // 32 * 32
        ck, cv = T.chunk_buffers(k, v, stride)
        kvx.append(tw.dev, 0, Gp.dev(ck), Gp.dev(cv), [td], [kvx.ChunkParams(done, n, stride, 129)],
                   H * stride * D)
        assert ko.store_chunk(ko.INT8, H, D, ck, cv, th,
                              ko.ChunkParams(done, n, stride, 129, tw.host.layer(0))) == 1
        done += n
    tw.assert_same_bytes()
    q = bf16_rows((1, H, 1, G, D), 2)
    splits = kvx.decode_plan([4096], H)
    got = decode_on_device(tw, 0, q, [td], [4096], [129], splits)
    want, want32 = decode_on_oracle(tw, 0, q, [th], [4096], [129], splits)
    Gp.check_attention(got, want, want32, np.ones((1, H), dtype=bool), tol(ko.INT8), "config 1")
    tw.close()


def test_config2_int4_long_context_batch1():
    # int4, batch 1, context 32768 behind a contiguous page table; one token is
    # appended, then attended.  Then the same pages behind shuffled page ids.
    committed, n_pages = 32768, 1025
    tw = Gp.Twin(ko.INT4, H, D, 2, 2 * n_pages, one_extent=True)
    pages = np.arange(n_pages, dtype=np.uint32)
    th, td = tw.tables(pages)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(2)
    device_history(tw, 1, td, n_pages, 0, committed, gen)
    device_history(tw, 1, td, n_pages, committed, 1, gen)      # the decode step's append
    tw.download()
    q = bf16_rows((1, H, 1, G, D), 3)
    splits = kvx.decode_plan([committed], H)
    assert 32 < splits[0] <= 512                               # the small-batch rule is in force
    got = decode_on_device(tw, 1, q, [td], [committed], [n_pages], splits)
    want, want32 = decode_on_oracle(tw, 1, q, [th], [committed], [n_pages], splits)
    stats = Gp.check_attention(got, want, want32, np.ones((1, H), dtype=bool), tol(ko.INT4),
                               "config 2",
                               explain=Gp.lanes_explainer(ko.INT4, H, G, D, q, [th], tw.host.layer(1),
                                                          [committed], 1, splits, 1, one_row=True))
    assert stats["rel_l2_mean"] < 1e-3
    # placement invariance: move every page to a shuffled id, attend again
    shuffled = (n_pages + np.random.default_rng(4).permutation(n_pages)).astype(np.uint32)
    tw.dev.copy_pages([(int(a), int(b)) for a, b in zip(pages, shuffled)])
    _, td2 = tw.tables(shuffled)
    again = decode_on_device(tw, 1, q, [td2], [committed], [n_pages], splits)
    assert np.array_equal(again, got)
    tw.close()


def test_config3_int4_mixed_batch32():
    # int4, batch 32, contexts U[512, 32768], shuffled pages of one pool; one
    # layer of the decode step against the oracle, every lane
    rng = np.random.default_rng(20261125)
    contexts = [int(c) for c in rng.integers(512, 32769, 32)]
    counts = [(c + 1 + 31) // 32 for c in contexts]
    tw = Gp.Twin(ko.INT4, H, D, 1, sum(counts), one_extent=True)
    ids = np.random.default_rng(5).permutation(sum(counts)).astype(np.uint32)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    hts, dts, first = [], [], 0
    for lane, n in enumerate(counts):
        th, td = tw.tables(ids[first:first + n])
        first += n
        hts.append(th)
        dts.append(td)
        device_history(tw, 0, td, n, 0, contexts[lane] + 1, gen)
    tw.download()
    q = bf16_rows((32, H, 1, G, D), 6)
    splits = kvx.decode_plan(contexts, H)
    got = decode_on_device(tw, 0, q, dts, contexts, counts, splits)
    want, want32 = decode_on_oracle(tw, 0, q, hts, contexts, counts, splits)
    stats = Gp.check_attention(got, want, want32, np.ones((32, H), dtype=bool), tol(ko.INT4),
                               "config 3",
                               explain=Gp.lanes_explainer(ko.INT4, H, G, D, q, hts, tw.host.layer(0),
                                                          contexts, 1, splits, 1, one_row=True))
    assert stats["rel_l2_mean"] < 5e-4
    tw.close()


@pytest.mark.parametrize("fmt", [ko.BF16, ko.FP8])
def test_config4_shared_prefix_chunked_prefill(fmt):
    # batch 4: a 16384-token prefix computed once and shared through the prefix
    # cache (512 whole pages), then a 2048-token chunk per sequence: quantize +
    # scatter, causal attention of 2048 rows over 18432 tokens
    prefix, chunk, sequences = 16384, 2048, 4
    prefix_pages, chunk_pages = prefix // 32, chunk // 32
    total_pages = prefix_pages + sequences * chunk_pages + prefix_pages   # + one private copy
    tw = Gp.Twin(fmt, H, D, 1, total_pages, one_extent=True)
    tw.dev.release(0)          # the pool allocates the device extent itself
    pool = kvx.Pool(tw.dev, tw.dev.page_count)
    cache = kvx.Prefix(pool)
    seqs = kvx.Sequences(pool, cache)
    tokens = [[(7 * i + 13 * s * (i >= prefix)) % 50021 for i in range(prefix + chunk)]
              for s in range(sequences)]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)
    # sequence 1 computes the prefix and publishes it
    seqs.begin(1)
    seqs.ensure_tokens(1, prefix + chunk)
    view = seqs.view(1)
    table1 = tw.dev.table(np.array(view["pages"], dtype=np.uint32))
    device_history(tw, 0, table1, len(view["pages"]), 0, prefix, gen)
    seqs.publish(1, tokens[0], prefix)
    # the others find it, adopt its pages and take pages of their own for the chunk
    tables = {1: table1}
    for s in range(2, sequences + 1):
        seqs.begin(s)
        blocks, hashed = cache.match(tokens[s - 1])
        assert len(blocks) == prefix_pages and hashed == prefix_pages + 1
        seqs.restore(s, blocks[-1])
        seqs.ensure_tokens(s, prefix + chunk)
        v = seqs.view(s)
        assert v["pages"][:prefix_pages] == view["pages"][:prefix_pages]
        assert not set(v["pages"][prefix_pages:]) & set(view["pages"])
        tables[s] = tw.dev.table(np.array(v["pages"], dtype=np.uint32))
    snap = pool.snapshot()
    assert snap.pages_prefix == prefix_pages
    assert snap.pages_active == prefix_pages + sequences * chunk_pages
    # every sequence appends its chunk and attends it
    n_entries = prefix_pages + chunk_pages
    splits = kvx.lib().kvx_prefill_splits(chunk)
    ws = torch.empty(kvx.prefill_workspace_bytes(tw.dev, chunk, QH) + 256, dtype=torch.uint8, device="cuda")
    outs, chunks, qs = {}, {}, {}
    for s in range(1, sequences + 1):
        k = torch.randn((H, chunk, D), generator=gen, device="cuda").bfloat16()
        v = torch.randn((H, D, chunk), generator=gen, device="cuda").bfloat16()
        q = torch.randn((H, chunk, G, D), generator=gen, device="cuda").bfloat16()
        chunks[s], qs[s] = (k, v), q
        kvx.append(tw.dev, 0, k, v, [tables[s]], [kvx.ChunkParams(prefix, chunk, chunk, n_entries)],
                   H * chunk * D)
        out = torch.zeros((H, chunk, G, D), dtype=torch.int16, device="cuda")
        kvx.attend_prefill(tw.dev, 0, QH, q, out, tables[s],
                           kvx.PrefillParams(prefix, chunk, chunk, n_entries, kvx.KvLayer(), splits, 0.0), ws)
        outs[s] = out
    torch.cuda.synchronize()
    # (a) shared pages against a private copy of the prefix: sequence 2 again,
    # with its prefix pages copied to fresh pages -- the bits must not change
    spare = pool.acquire(prefix_pages)
    shared = seqs.view(2)["pages"]
    tw.dev.copy_pages(list(zip(shared[:prefix_pages], spare)))
    private = tw.dev.table(np.array(spare + shared[prefix_pages:], dtype=np.uint32))
    out_private = torch.zeros((H, chunk, G, D), dtype=torch.int16, device="cuda")
    kvx.attend_prefill(tw.dev, 0, QH, qs[2], out_private, private,
                       kvx.PrefillParams(prefix, chunk, chunk, n_entries, kvx.KvLayer(), splits, 0.0), ws)
    torch.cuda.synchronize()
    assert torch.equal(out_private, outs[2])
    # the copies are byte-identical and the sources untouched
    for a, b in list(zip(shared[:prefix_pages], spare))[::97]:
        assert np.array_equal(tw.dev.page_read(a), tw.dev.page_read(b))
    # (b) the oracle on sampled tiles of sequence 2: first, middle, last
    tw.download()
    table_host = tw.host.entries(np.array(shared, dtype=np.uint32))
    q_host = Gp.host_u16(qs[2].view(torch.int16))
    got = Gp.host_u16(outs[2])
    rels = []
    for tile in (0, 127, 255):
        for head in (0, 3):
            tile_q = q_host[head, 8 * tile:8 * tile + 8].reshape(8 * G, D)
            want, want32 = Gp.oracle_tile(fmt, H, G, D, tile_q, table_host, tw.host.layer(0), head,
                                          prefix + 8 * tile, 8, splits, 8)
            mine = got[head, 8 * tile:8 * tile + 8].reshape(8 * G, D)
            stats = Gp.check_attention(
                mine, want, want32, np.ones(8 * G, dtype=bool), tol(fmt),
                f"config 4 fmt={fmt} tile {tile} head {head}",
                explain=lambda index: dict(fmt=fmt, kv_heads=H, group=G, head_dim=D, tile_queries=tile_q,
                                           table=table_host, kv=tw.host.layer(0), head=head,
                                           committed=prefix + 8 * tile, active=8, splits=splits,
                                           capacity=8, fused_row=index[0]))
            rels.append(stats["rel_l2_mean"])
    assert np.mean(rels) < (4e-3 if fmt == ko.FP8 else 1e-3)
    for s in range(1, sequences + 1):
        seqs.end(s)
    for p in spare:
        pool.release(p)
    assert pool.snapshot().pages_active == 0 and pool.snapshot().pages_prefix == prefix_pages
    seqs.close()
    cache.close()
    pool.close()
    tw.close()


@pytest.mark.parametrize("fmt", [ko.BF16, ko.FP8, ko.INT4])
def test_config4_copy_on_write_of_the_partial_last_page(fmt):
    """configs[3] with a prefix that does not end on a page boundary: 16 400 tokens = 512 whole
    pages and 16 tokens of a 513th.  The second sequence forks the first at 16 400 tokens (every
    page shared by reference, the partial one included), and its first store triggers the copy:
    kv_page_copy of the partial page, every layer, into a page of its own, then the chunk's rows
    from slot 16 on.  The reference shares whole pages only (runtime/engine/cache/Cache.cpp:183-184,
    :774), so the pins are invariants: the copy is the source's bytes, the source is untouched,
    the references add up, and after the store every byte equals the oracle's page copy + store."""
    prefix, chunk, layers = 16400, 2048, 2
    whole = prefix // 32
    prefix_pages, total_pages = whole + 1, whole + 1 + 2 * ((prefix % 32 + chunk + 31) // 32) + 8
    tw = Gp.Twin(fmt, H, D, layers, total_pages, one_extent=True)
    tw.dev.release(0)                      # the pool allocates the device extent itself
    pool = kvx.Pool(tw.dev, tw.dev.page_count)
    cache = kvx.Prefix(pool)
    seqs = kvx.Sequences(pool, cache)
    gen = torch.Generator(device="cuda").manual_seed(44)
    tokens = [(11 * i) % 50021 for i in range(prefix + chunk)]
    # the first sequence computes the prefix and publishes its whole pages
    seqs.begin(1)
    seqs.ensure_tokens(1, prefix)
    one = seqs.view(1)
    assert len(one["pages"]) == prefix_pages
    table1 = tw.dev.table(np.array(one["pages"], dtype=np.uint32))
    for layer in range(layers):
        device_history(tw, layer, table1, prefix_pages, 0, prefix, gen, outliers=True)
    torch.cuda.synchronize()
    seqs.publish(1, tokens, prefix)
    assert len(seqs.view(1)["blocks"]) == whole
    # the fork: all 513 pages by reference, no copy yet
    seqs.begin(2)
    seqs.fork(2, 1, prefix)
    two = seqs.view(2)
    assert two["pages"] == one["pages"] and two["blocks"] == seqs.view(1)["blocks"]
    snap = pool.snapshot()
    assert snap.pages_active == prefix_pages and snap.pages_prefix == whole
    partial = one["pages"][whole]
    source_bytes = tw.dev.page_read(partial)
    assert source_bytes.any()
    tw.download()                          # the oracle's store takes over the history so far
    # the fork's first store: copy-on-write of the partial page, then pages for the chunk
    moved = seqs.ensure_writable(2, prefix)
    assert moved is not None and moved[0] == partial and moved[1] not in one["pages"]
    copy = moved[1]
    torch.cuda.synchronize()
    assert np.array_equal(tw.dev.page_read(copy), source_bytes)        # every layer, every tensor
    seqs.ensure_tokens(2, prefix + chunk)
    two = seqs.view(2)
    assert two["pages"][:whole] == one["pages"][:whole] and two["pages"][whole] == copy
    assert not set(two["pages"][whole:]) & set(one["pages"])
    assert two["first_changed"] == prefix_pages and two["revision"] == 3
    n_entries = len(two["pages"])
    snap = pool.snapshot()
    assert snap.pages_active == prefix_pages + (n_entries - whole) and snap.pages_prefix == whole
    assert all(pool.page_active(p) for p in one["pages"] + two["pages"])
    # the oracle's side: its own whole-page copy, after which both stores hold the same bytes
    assert tw.host.copy_pages([(partial, copy)]) == 0
    tw.assert_same_bytes()
    table2 = tw.dev.table(np.array(two["pages"], dtype=np.uint32))
    table2_host = tw.host.entries(np.array(two["pages"], dtype=np.uint32))
    k = torch.randn((H, chunk, D), generator=gen, device="cuda").bfloat16()
    v = torch.randn((H, D, chunk), generator=gen, device="cuda").bfloat16()
    for layer in range(layers):
        kvx.append(tw.dev, layer, k, v, [table2], [kvx.ChunkParams(prefix, chunk, chunk, n_entries)],
                   H * chunk * D)
        p = ko.ChunkParams(prefix, chunk, chunk, n_entries, tw.host.layer(layer))
        assert ko.store_chunk(fmt, H, D, Gp.host_u16(k.view(torch.int16)),
                              Gp.host_u16(v.view(torch.int16)), table2_host, p) == 1
    torch.cuda.synchronize()
    tw.assert_same_bytes()                                             # copy + store, bit for bit
    assert np.array_equal(tw.dev.page_read(partial), source_bytes)     # the shared page is untouched
    # the copy: slots 0..15 are the source's rows, slots 16..31 the chunk's first rows
    assert not np.array_equal(tw.dev.page_read(copy), source_bytes)
    # attention of the chunk over prefix + chunk through the fork's table, sampled tiles
    q = torch.randn((H, chunk, G, D), generator=gen, device="cuda").bfloat16()
    splits = kvx.lib().kvx_prefill_splits(chunk)
    ws = torch.empty(kvx.prefill_workspace_bytes(tw.dev, chunk, QH) + 256, dtype=torch.uint8, device="cuda")
    out = torch.zeros((H, chunk, G, D), dtype=torch.int16, device="cuda")
    kvx.attend_prefill(tw.dev, 1, QH, q, out, table2,
                       kvx.PrefillParams(prefix, chunk, chunk, n_entries, kvx.KvLayer(), splits, 0.0), ws)
    torch.cuda.synchronize()
    q_host, got = Gp.host_u16(q.view(torch.int16)), Gp.host_u16(out)
    for tile, head in ((0, 0), (1, 2), (255, 3)):
        tile_q = q_host[head, 8 * tile:8 * tile + 8].reshape(8 * G, D)
        want, want32 = Gp.oracle_tile(fmt, H, G, D, tile_q, table2_host, tw.host.layer(1), head,
                                      prefix + 8 * tile, 8, splits, 8)
        mine = got[head, 8 * tile:8 * tile + 8].reshape(8 * G, D)
        Gp.check_attention(
            mine, want, want32, np.ones(8 * G, dtype=bool), tol(fmt),
            f"config 4 copy-on-write fmt={fmt} tile {tile} head {head}",
            explain=lambda index: dict(fmt=fmt, kv_heads=H, group=G, head_dim=D, tile_queries=tile_q,
                                       table=table2_host, kv=tw.host.layer(1), head=head,
                                       committed=prefix + 8 * tile, active=8, splits=splits,
                                       capacity=8, fused_row=index[0]))
    # the source goes on writing its own page in place; the references unwind
    assert seqs.ensure_writable(1, prefix) is None
    seqs.end(1)
    assert all(pool.page_active(p) for p in two["pages"]) and not pool.page_active(partial)
    seqs.end(2)
    snap = pool.snapshot()
    assert snap.pages_active == 0 and snap.pages_prefix == whole
    seqs.close()
    cache.close()
    pool.close()
    tw.close()


@pytest.mark.parametrize("rule", ["reference", "plan"])
def test_config5_int4_tree_verify_and_rollback(rule):
    """int4, batch 4, contexts of 65 536 tokens (two a little further, so that their 16 draft
    rows run over a page boundary), a 16-row tree per sequence: append the rows, masked verify
    under the reference's split rule and under kvx_verify_plan (what bench.py and the
    integration notes use), a root-to-leaf path per sequence, compaction; the page bytes after
    the rollback must be the oracle's, bit for bit.  The pages come from the pool through the
    sequence records: after the rollback kvx_sequence_truncate gives the page that holds only
    rejected rows back, the pool's counts and the page lists say so, and the next step's rows
    land in the slots behind the accepted ones."""
    lanes, nodes = 4, 16
    committed = [65536, 65560, 65556, 65536]
    n_pages = [(c + nodes + 31) // 32 for c in committed]
    tw = Gp.Twin(ko.INT4, H, D, 1, sum(n_pages) + 8, one_extent=True)
    tw.dev.release(0)                      # the pool allocates the device extent itself
    pool = kvx.Pool(tw.dev, tw.dev.page_count)
    cache = kvx.Prefix(pool)
    seqs = kvx.Sequences(pool, cache)
    # page ids in a seed-shuffled order: everything acquired once and given back shuffled,
    # so that the sequences' pages come off the free stacks scattered over the extent
    every = pool.acquire(sum(n_pages) + 4)
    for page in np.random.default_rng(8).permutation(every):
        pool.release(int(page))
    assert pool.snapshot().pages_active == 0
    gen = torch.Generator(device="cuda")
    gen.manual_seed(8)
    hts, dts = [], []
    for lane in range(lanes):
        seqs.begin(lane + 1)
        seqs.ensure_tokens(lane + 1, committed[lane] + nodes)
        pages = np.array(seqs.view(lane + 1)["pages"], dtype=np.uint32)
        assert len(pages) == n_pages[lane] and len(set(np.diff(pages.astype(np.int64)))) > 100
        th, td = tw.tables(pages)
        hts.append(th)
        dts.append(td)
        device_history(tw, 0, td, n_pages[lane], 0, committed[lane], gen)
    held = pool.snapshot().pages_active
    assert held == sum(n_pages)
    tw.download()
    rng = np.random.default_rng(9)
    none = 0xFFFFFFFF
    parents, masks = [], np.zeros((lanes, nodes), dtype=np.uint32)
    for lane in range(lanes):
        # topologically ordered, branching at most 3
        p, children = [none], {0: 0}
        for row in range(1, nodes):
            choices = [c for c in range(row) if children.get(c, 0) < 3]
            parent = int(rng.choice(choices[-4:]))
            children[parent] = children.get(parent, 0) + 1
            p.append(parent)
        parents.append(p)
        masks[lane] = kvx.tree_masks(p)
    # the rows' K/V go through the verify store on both sides
    k = rng.standard_normal((lanes, H, nodes, D)).astype(np.float32)
    v = rng.standard_normal((lanes, H, nodes, D)).astype(np.float32)
    ck = np.zeros((lanes, H, 32, D), dtype=np.uint16)
    cv = np.zeros((lanes, H, D, 32), dtype=np.uint16)
    for lane in range(lanes):
        ck[lane], cv[lane] = T.chunk_buffers(k[lane], v[lane], 32)
    dparams = [kvx.ChunkParams(committed[i], nodes, 32, n_pages[i]) for i in range(lanes)]
    kvx.append(tw.dev, 0, Gp.dev(ck), Gp.dev(cv), dts, dparams, H * 32 * D, verify_max_rows=16)
    hparams = [ko.ChunkParams(committed[i], nodes, 32, n_pages[i], tw.host.layer(0)) for i in range(lanes)]
    assert ko.store_verify(ko.INT4, H, D, ck, cv, hts, hparams, max_rows=16) == lanes
    # masked verify on the device; the oracle on one lane, two heads
    q = np.zeros((lanes, H, 32, G, D), dtype=np.uint16)
    q[:, :, :nodes] = bf16_rows((lanes, H, nodes, G, D), 10)
    if rule == "reference":
        splits = [kvx.lib().kvx_verify_splits(c, nodes) for c in committed]
        assert splits == [128] * lanes
    else:
        splits = kvx.verify_plan(committed, nodes, H, QH)
        # three waves of 32 fused rows per split and KV head, one round of the 1024 SIMDs
        assert splits == [21] * lanes and sum(splits) * H * 3 <= 1024
    dp = [kvx.VerifyParams(committed[i], n_pages[i], kvx.KvLayer(), splits[i], 128, nodes, 16, 0.0)
          for i in range(lanes)]
    out = torch.zeros((lanes, H, 32, G, D), dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH) + 256, dtype=torch.uint8, device="cuda")
    kvx.attend_verify(tw.dev, 0, QH, Gp.dev(q), out, dts, dp, Gp.dev(masks), 32, ws)
    torch.cuda.synchronize()
    got = Gp.host_u16(out)
    for lane, heads in ((2, (0, 3)), (1, (2,))):
        for head in heads:
            tile_q = q[lane, head, :16].reshape(16 * G, D)
            want, want32 = Gp.oracle_tile(ko.INT4, H, G, D, tile_q, hts[lane], tw.host.layer(0), head,
                                          committed[lane], nodes, splits[lane], 16, masks=masks[lane])
            mine = got[lane, head, :16].reshape(16 * G, D)
            Gp.check_attention(
                mine, want, want32, np.ones(16 * G, dtype=bool), tol(ko.INT4),
                f"config 5 ({rule} splits) lane {lane} head {head}",
                explain=lambda index: dict(fmt=ko.INT4, kv_heads=H, group=G, head_dim=D,
                                           tile_queries=tile_q, table=hts[lane], kv=tw.host.layer(0),
                                           head=head, committed=committed[lane], active=nodes,
                                           splits=splits[lane], capacity=16, fused_row=index[0],
                                           masks=masks[lane]))
    # a tree that is a path must see exactly what the chain sees
    chain_masks = np.zeros((lanes, nodes), dtype=np.uint32)
    chain_masks[:] = kvx.tree_masks([none] + list(range(nodes - 1)))
    out_path = torch.zeros_like(out)
    kvx.attend_verify(tw.dev, 0, QH, Gp.dev(q), out_path, dts, dp, Gp.dev(chain_masks), 32, ws)
    out_chain = torch.zeros_like(out)
    kvx.attend_verify(tw.dev, 0, QH, Gp.dev(q), out_chain, dts, dp, None, 32, ws)
    torch.cuda.synchronize()
    assert torch.equal(out_path, out_chain)
    # acceptance: a seeded root-to-leaf walk per sequence; then compaction
    paths = np.zeros((lanes, 16), dtype=np.uint32)
    counts = np.zeros(lanes, dtype=np.uint32)
    for i in range(lanes):
        walk, row = [0], 0
        while True:
            kids = [c for c in range(nodes) if parents[i][c] == row]
            if not kids:
                break
            row = int(rng.choice(kids))
            walk.append(row)
        assert kvx.tree_path_valid(parents[i], walk)
        paths[i, :len(walk)] = walk
        counts[i] = len(walk)
    kvx.compact_path(tw.dev, 0, dts, dparams, Gp.dev(paths), Gp.dev(counts), 16)
    torch.cuda.synchronize()
    assert ko.compact_tree(ko.INT4, H, D, hts, hparams, paths, counts, 16) > 0   # rows moved
    tw.assert_same_bytes()
    # the rollback frees what it emptied: the host's committed count moves on by the accepted
    # rows, and a page none of them reached goes back to the pool
    after = [committed[i] + int(counts[i]) for i in range(lanes)]
    emptied = [n_pages[i] - (after[i] + 31) // 32 for i in range(lanes)]
    assert sum(emptied) >= 1 and emptied[0] == 0 and emptied[3] == 0   # page-aligned lanes keep theirs
    for i in range(lanes):
        before = seqs.view(i + 1)
        assert seqs.truncate(i + 1, after[i]) == emptied[i]
        view = seqs.view(i + 1)
        assert view["pages"] == before["pages"][:n_pages[i] - emptied[i]]
        if emptied[i]:
            dropped = before["pages"][-1]
            assert not pool.page_active(dropped)
            assert view["revision"] == before["revision"] + 1
            assert view["first_changed"] == len(view["pages"])
    assert pool.snapshot().pages_active == held - sum(emptied)
    # the next step: room for another tree, its rows stored behind the accepted ones
    k2 = rng.standard_normal((lanes, H, nodes, D)).astype(np.float32)
    v2 = rng.standard_normal((lanes, H, nodes, D)).astype(np.float32)
    for lane in range(lanes):
        ck[lane], cv[lane] = T.chunk_buffers(k2[lane], v2[lane], 32)
    hts2, dts2, next_pages = [], [], []
    for lane in range(lanes):
        seqs.ensure_tokens(lane + 1, after[lane] + nodes)
        pages = np.array(seqs.view(lane + 1)["pages"], dtype=np.uint32)
        next_pages.append(len(pages))
        assert len(pages) == (after[lane] + nodes + 31) // 32
        th, td = tw.tables(pages)
        hts2.append(th)
        dts2.append(td)
    assert pool.snapshot().pages_active == sum(next_pages)
    dparams2 = [kvx.ChunkParams(after[i], nodes, 32, next_pages[i]) for i in range(lanes)]
    kvx.append(tw.dev, 0, Gp.dev(ck), Gp.dev(cv), dts2, dparams2, H * 32 * D, verify_max_rows=16)
    torch.cuda.synchronize()
    hparams2 = [ko.ChunkParams(after[i], nodes, 32, next_pages[i], tw.host.layer(0)) for i in range(lanes)]
    assert ko.store_verify(ko.INT4, H, D, ck, cv, hts2, hparams2, max_rows=16) == lanes
    tw.assert_same_bytes()
    for lane in range(lanes):
        seqs.end(lane + 1)
    assert pool.snapshot().pages_active == 0
    seqs.close()
    cache.close()
    pool.close()
    tw.close()
