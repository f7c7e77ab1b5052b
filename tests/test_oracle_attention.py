"""Oracle attention: pinned to tolerance by dense fp64 softmax, special cases
that reduce to closed forms, the reference tests' own integer patterns and
gates (dev/tests/engine/paged_attention_plan_test.mm:358-501, :1018-1029) and
its merge test (dev/tests/engine/q8_flash_attention_metal_test.mm:648-725).

Bit-level parity with the Metal kernels is unpinned: their exp and matmul
order live in Apple's runtime.  Tree verify has no reference test at all and
is pinned here by brute force only.
"""
import ctypes as C

import numpy as np
import pytest

from oracle import kvoracle as ko
import kvtestlib as T

L = ko.lib()
H, G, D = 4, 6, 256
FORMATS = [ko.INT8, ko.INT4, ko.BF16, ko.FP8]


def build_history(fmt, committed, rows, seed, lane=0, pattern=False, layers=2, layer=1,
                  one_extent=False, scale=1.0):
    """Appends committed+rows tokens through the oracle store; returns
    (store, pages, table, K, V) with K/V the dequantisable code views."""
    total = committed + rows
    n_pages = (total + 31) // 32
    store = T.make_store(fmt, H, D, layers, n_pages, one_extent)
    pages = T.mixed_pages(store.extent_pages, store.page_count // store.extent_pages, n_pages, seed)
    table = store.entries(pages)
    rng = np.random.default_rng(seed)
    done = 0
    while done < total:
        n = min(2048, total - done)
        k = (rng.standard_normal((H, n, D)) * scale).astype(np.float32)
        v = (rng.standard_normal((H, n, D)) * scale).astype(np.float32)
        stride = (n + 31) // 32 * 32
        ck, cv = T.chunk_buffers(k, v, stride)
        p = ko.ChunkParams(done, n, stride, n_pages, store.layer(layer))
        assert ko.store_chunk(fmt, H, D, ck, cv, table, p) == 1
        done += n
    return store, pages, table


def history_codes(store, pages, layer, tokens):
    parts = [T.page_codes(store, layer, int(p)) for p in pages]
    kc = np.concatenate([x[0] for x in parts], axis=1)[:, :tokens]
    ks = np.concatenate([x[1] for x in parts], axis=1)[:, :tokens]
    vc = np.concatenate([x[2] for x in parts], axis=1)[:, :tokens]
    vs = np.concatenate([x[3] for x in parts], axis=1)[:, :tokens]
    return kc, ks, vc, vs


def random_queries(rows, stride, seed, scale=1.0):
    rng = np.random.default_rng(seed + 1000)
    q = np.zeros((H, stride, G, D), dtype=np.uint16)
    q[:, :rows] = ko.f32_to_bf16((rng.standard_normal((H, rows, G, D)) * scale).astype(np.float32)
                                 ).reshape(H, rows, G, D)
    return q


def dense_reference(fmt, q, kc, ks, vc, vs, committed, rows, score_scale=0.0625):
    out = np.zeros((H, rows, G, D))
    for h in range(H):
        qq = ko.bf16_to_f32(q[h, :rows]).reshape(rows * G, D)
        if fmt == ko.FP8:
            qq = qq.astype(np.float16).astype(np.float32)
        limits = np.repeat(committed + np.arange(rows) + 1, G)
        out[h] = T.dense_attention_f64(qq, kc[h], ks[h], vc[h], vs[h], limits,
                                       score_scale).reshape(rows, G, D)
    return out


def gates(got, want):
    got, want = got.reshape(-1).astype(np.float64), want.reshape(-1).astype(np.float64)
    cos = got @ want / np.sqrt((got @ got) * (want @ want))
    return np.abs(got - want).max(), cos


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("committed,rows", [(0, 1), (33, 7), (255, 17), (1023, 8), (100, 77)])
def test_prefill_against_dense_fp64(fmt, committed, rows):
    store, pages, table = build_history(fmt, committed, rows, seed=committed + rows)
    stride = (rows + 31) // 32 * 32
    q = random_queries(rows, stride, committed)
    tiles = (rows + 7) // 8
    p = ko.PrefillParams(committed, rows, stride, len(pages), store.layer(1),
                         L.ko_prefill_splits(tiles), 0.0)
    ok, out, f32 = ko.attend_prefill(fmt, H, G, D, q, table, p)
    assert ok == 1
    kc, ks, vc, vs = history_codes(store, pages, 1, committed + rows)
    want = dense_reference(fmt, q, kc, ks, vc, vs, committed, rows)
    # the bf16 (fp16) rounding of probability x value scale is the only
    # departure from exact softmax: the reference's own gates bound it
    err, cos = gates(f32[:, :rows], want)
    assert err < 0.02 and cos > (0.998 if fmt == ko.INT4 else 0.9995)
    assert T.rel_l2(f32[:, :rows], want).max() < (1e-2 if fmt == ko.FP8 else 4e-3)
    # the bf16 output is the rounding of the fp32 one; padding rows stay zero
    assert np.array_equal(out, ko.f32_to_bf16(f32).reshape(out.shape))
    assert not out[:, rows:].any()


@pytest.mark.parametrize("fmt", [ko.INT8, ko.INT4, ko.BF16])
@pytest.mark.parametrize("committed,rows", [(0, 1), (33, 7), (255, 17), (1023, 8)])
def test_reference_plan_test_patterns_and_gates(fmt, committed, rows):
    """Integer code patterns with fixed scales written straight into the pages
    and checked with the reference's checkReference fold order and gates."""
    int4 = fmt == ko.INT4
    total = committed + rows
    n_pages = (total + 31) // 32
    store = T.make_store(fmt, H, D, 2, n_pages)
    pages = T.mixed_pages(store.extent_pages, store.page_count // store.extent_pages, n_pages,
                          committed + rows + 1)
    table = store.entries(pages)
    tok, hh, dd = np.meshgrid(np.arange(total), np.arange(H), np.arange(D), indexing="ij")
    kcode = T.plan_key_code(tok, hh, dd, 0, int4).astype(np.float32)    # [T][H][D]
    vcode = T.plan_value_code(tok, hh, dd, 0, int4).astype(np.float32)
    kscale, vscale = (0.096, 0.112) if int4 else (0.006, 0.007)
    for pi, page in enumerate(pages):
        k, ks, v, vs = T.slab_views(store, 1, int(page))
        n = min(32, total - pi * 32)
        kk = np.zeros((H, 32, D), dtype=np.float32)
        vv = np.zeros((H, 32, D), dtype=np.float32)
        kk[:, :n] = kcode[pi * 32:pi * 32 + n].transpose(1, 0, 2)
        vv[:, :n] = vcode[pi * 32:pi * 32 + n].transpose(1, 0, 2)
        if fmt == ko.INT4:
            ki, vi = kk.astype(np.int32), vv.astype(np.int32)
            k[:] = ((ki[..., 0::2] & 0xF) | ((ki[..., 1::2] & 0xF) << 4)).astype(np.uint8).reshape(-1)
            v[:] = ((vi[..., 0::2] & 0xF) | ((vi[..., 1::2] & 0xF) << 4)).astype(np.uint8).reshape(-1)
        elif fmt == ko.INT8:
            k[:] = kk.astype(np.int8).view(np.uint8).reshape(-1)
            v[:] = vv.transpose(0, 2, 1).astype(np.int8).view(np.uint8).reshape(-1)
        else:
            k[:] = ko.f32_to_bf16(kk * np.float32(0.006)).view(np.uint8).reshape(-1)
            v[:] = ko.f32_to_bf16(vv.transpose(0, 2, 1) * np.float32(0.007)).view(np.uint8).reshape(-1)
        if fmt != ko.BF16:
            ks.view(np.float32)[:] = kscale
            vs.view(np.float32)[:] = vscale
    stride = (rows + 31) // 32 * 32
    r, qh, d3 = np.meshgrid(np.arange(rows), np.arange(H * G), np.arange(D), indexing="ij")
    qv = T.plan_query(r, qh, d3).astype(np.float32)  # [row][qhead][D]
    q = np.zeros((H, stride, G, D), dtype=np.uint16)
    q[:, :rows] = ko.f32_to_bf16(qv).reshape(rows, H, G, D).transpose(1, 0, 2, 3)
    p = ko.PrefillParams(committed, rows, stride, n_pages, store.layer(1),
                         L.ko_prefill_splits((rows + 7) // 8), 0.0)
    ok, out, f32 = ko.attend_prefill(fmt, H, G, D, q, table, p)
    assert ok == 1
    kc, ks_, vc, vs_ = history_codes(store, pages, 1, total)
    got = ko.bf16_to_f32(out).reshape(out.shape)
    gots, wants = [], []  # one cosine over every sampled row, as checkReference does
    for row in sorted({0, min(7, rows - 1), rows // 2, rows - 1}):
        for head in (0, H * G - 1):
            kvh, g = head // G, head % G
            n = committed + row + 1
            qq = ko.bf16_to_f32(q[kvh, row, g]).astype(np.float32)
            # fp32, raw-code dot then one multiply by the token scale
            s = (kc[kvh, :n] @ qq).astype(np.float32) * ks_[kvh, :n] * np.float32(0.0625)
            e = np.exp(s - s.max()).astype(np.float32)
            want = ((e * vs_[kvh, :n]) @ vc[kvh, :n]) / e.sum()
            gots.append(got[kvh, row, g])
            wants.append(want)
    err, cos = gates(np.concatenate(gots), np.concatenate(wants))
    assert err < 0.02 and cos > (0.998 if int4 else 0.9995)


@pytest.mark.parametrize("fmt", FORMATS)
def test_single_token_returns_its_value_row(fmt):
    store, pages, table = build_history(fmt, 0, 1, seed=4)
    q = random_queries(1, 32, 4)
    p = ko.PrefillParams(0, 1, 32, 1, store.layer(1), 32, 0.0)
    ok, out, f32 = ko.attend_prefill(fmt, H, G, D, q, table, p)
    kc, ks, vc, vs = history_codes(store, pages, 1, 1)
    for h in range(H):
        w = np.float32(vs[h, 0])
        w = np.float16(w).astype(np.float32) if fmt == ko.FP8 else ko.bf16_to_f32(ko.f32_to_bf16(w))[()]
        for g in range(G):
            assert np.array_equal(f32[h, 0, g], (w * vc[h, 0]).astype(np.float32))


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16])
def test_zero_query_gives_the_mean_value(fmt):
    committed, rows = 95, 1
    store, pages, table = build_history(fmt, committed, rows, seed=8)
    q = np.zeros((H, 32, G, D), dtype=np.uint16)
    p = ko.PrefillParams(committed, rows, 32, len(pages), store.layer(1), 1, 0.0)
    ok, out, f32 = ko.attend_prefill(fmt, H, G, D, q, table, p)
    kc, ks, vc, vs = history_codes(store, pages, 1, committed + rows)
    for h in range(H):
        w = ko.bf16_to_f32(ko.f32_to_bf16(vs[h])).astype(np.float64)
        want = (w[:, None] * vc[h]).sum(axis=0) / (committed + rows)
        assert np.allclose(f32[h, 0, 0], want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("fmt", [ko.INT4, ko.BF16])
def test_split_count_only_perturbs_rounding(fmt):
    # A different partition moves each page's running maximum, and with it the
    # point at which probability x value scale is rounded to bf16: the results
    # differ by that rounding's noise (about 2^-9 / sqrt(tokens)), not more.
    committed, rows = 1500, 3
    store, pages, table = build_history(fmt, committed, rows, seed=15)
    q = random_queries(rows, 32, 15)
    outs = []
    for splits in (1, 3, 32):
        p = ko.PrefillParams(committed, rows, 32, len(pages), store.layer(1), splits, 0.0)
        outs.append(ko.attend_prefill(fmt, H, G, D, q, table, p)[2])
    for o in outs[1:]:
        assert T.rel_l2(o[:, :rows], outs[0][:, :rows]).max() < 5e-3


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8])
def test_extents_do_not_change_bits(fmt):
    # dev/tests/engine/q8_flash_attention_metal_test.mm:634-640
    committed, rows = 300, 9
    res = []
    for one in (False, True):
        store, pages, table = build_history(fmt, committed, rows, seed=21, one_extent=one)
        q = random_queries(rows, 32, 21)
        p = ko.PrefillParams(committed, rows, 32, len(pages), store.layer(1), 16, 0.0)
        res.append(ko.attend_prefill(fmt, H, G, D, q, table, p)[1])
    assert np.array_equal(res[0], res[1])


def verify_case(fmt, committed_list, active, capacity, seed, masks=None):
    lanes = len(committed_list)
    stores, tables, params = [], [], []
    for lane, committed in enumerate(committed_list):
        store, pages, table = build_history(fmt, committed, active, seed=seed + lane)
        stores.append((store, pages))
        tables.append(table)
        splits = L.ko_verify_splits(committed, active)
        params.append(ko.VerifyParams(committed, len(pages), store.layer(1), splits, 128, active,
                                      capacity, 0.0))
    rng = np.random.default_rng(seed)
    q = np.zeros((lanes, H, 32, G, D), dtype=np.uint16)
    q[:, :, :capacity] = ko.f32_to_bf16(rng.standard_normal((lanes, H, capacity, G, D)).astype(np.float32)
                                        ).reshape(lanes, H, capacity, G, D)
    n, out, f32 = ko.attend_verify(fmt, H, G, D, q, tables, params, masks)
    assert n == lanes
    return stores, tables, params, q, out, f32


@pytest.mark.parametrize("fmt", [ko.INT8, ko.INT4, ko.BF16, ko.FP8])
def test_verify_chain_against_dense_fp64(fmt):
    committed_list = [0, 1023, 1023 + 649]
    stores, tables, params, q, out, f32 = verify_case(fmt, committed_list, 8, 8, seed=31)
    for lane, committed in enumerate(committed_list):
        store, pages = stores[lane]
        kc, ks, vc, vs = history_codes(store, pages, 1, committed + 8)
        want = dense_reference(fmt, q[lane], kc, ks, vc, vs, committed, 8)
        assert T.rel_l2(f32[lane][:, :8], want).max() < (1e-2 if fmt == ko.FP8 else 4e-3)
        assert not out[lane][:, 8:].any()


def test_verify_matches_prefill_bits_for_the_same_partition():
    # dev/tests/engine/q8_flash_attention_metal_test.mm:786-793
    committed = 777
    stores, tables, params, q, out, f32 = verify_case(ko.INT4, [committed], 8, 8, seed=41)
    store, pages = stores[0]
    p = ko.PrefillParams(committed, 8, 32, len(pages), store.layer(1), 32, 0.0)
    ok, pout, pf32 = ko.attend_prefill(ko.INT4, H, G, D, q[0], tables[0], p)
    assert params[0].split_count == 32 and np.array_equal(pout, out[0])


def tree_masks(parents):
    """Ancestor bitmasks (self included) of a topologically ordered tree:
    shared/embedding.metal:248-281 builds mask = 1<<row | ancestors."""
    masks = []
    for row, parent in enumerate(parents):
        masks.append((1 << row) | (masks[parent] if parent >= 0 else 0))
    return masks


def test_tree_with_path_masks_equals_chain():
    committed = 500
    chain = verify_case(ko.INT4, [committed], 8, 8, seed=51)
    masks = np.zeros((1, 16), dtype=np.uint32)
    masks[0, :8] = tree_masks([-1, 0, 1, 2, 3, 4, 5, 6])
    lanes_q = np.zeros((1, H, 32, G, D), dtype=np.uint16)
    lanes_q[:, :, :8] = chain[3][:, :, :8]
    store, pages = chain[0][0]
    p = ko.VerifyParams(committed, len(pages), store.layer(1), chain[2][0].split_count, 128, 8, 16, 0.0)
    n, out, f32 = ko.attend_verify(ko.INT4, H, G, D, lanes_q, chain[1], [p], masks)
    assert n == 1 and np.array_equal(out[:, :, :8], chain[4][:, :, :8])
    assert not out[:, :, 8:].any()


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16])
def test_tree_masks_against_dense_fp64(fmt):
    committed, nodes = 260, 16
    parents = [-1, 0, 0, 1, 1, 2, 3, 3, 3, 5, 6, 8, 8, 9, 11, 12]
    masks = np.array([tree_masks(parents)], dtype=np.uint32)
    stores, tables, params, q, out, f32 = verify_case(fmt, [committed], nodes, 16, seed=61, masks=masks)
    store, pages = stores[0]
    kc, ks, vc, vs = history_codes(store, pages, 1, committed + nodes)
    T_all = committed + nodes
    admit = np.zeros((nodes, T_all), dtype=bool)
    admit[:, :committed] = True
    for row in range(nodes):
        for j in range(nodes):
            admit[row, committed + j] = (masks[0, row] >> j) & 1
    for h in range(H):
        qq = ko.bf16_to_f32(q[0, h, :nodes]).reshape(nodes * G, D)
        want = T.dense_attention_f64(qq, kc[h], ks[h], vc[h], vs[h], np.repeat(admit, G, axis=0), 0.0625)
        assert T.rel_l2(f32[0, h, :nodes].reshape(nodes * G, D), want).max() < 4e-3


def test_invalid_verify_lane_writes_nothing():
    stores, tables, params, q, out, f32 = verify_case(ko.INT8, [40, 40], 8, 8, seed=71)
    params[1].page_table_entries = 1
    n, out2, _ = ko.attend_verify(ko.INT8, H, G, D, q, tables, params, None)
    assert n == 1 and np.array_equal(out2[0], out[0]) and not out2[1].any()
    bad = ko.PrefillParams(40, 8, 32, 1, stores[0][0].layer(1), 4, 0.0)
    ok, o, _ = ko.attend_prefill(ko.INT8, H, G, D, q[0], tables[0], bad)
    assert ok == 0 and not o.any()


@pytest.mark.parametrize("splits,active", [(1, 8), (5, 8), (32, 8), (128, 8), (7, 3), (32, 1)])
def test_merge_against_fp64_reference_pattern(splits, active):
    m = 8 * G
    s_idx, r_idx = np.meshgrid(np.arange(splits), np.arange(m), indexing="ij")
    act = (r_idx // G) < active
    spacing = np.where(r_idx % 2 == 1, 0.25, 500.0)
    mx = np.where(act, ((s_idx % 5) - 2) * spacing, -np.inf).astype(np.float32)
    sm = np.where(act, 1.0 + (s_idx % 7), 0.0).astype(np.float32)
    stats = np.stack([mx, sm], axis=-1).astype(np.float32).copy()           # [split][row][2]
    d_idx = np.arange(D)
    part = (((s_idx[..., None] * 71 + d_idx * 37 + r_idx[..., None] * 13) % 257) - 128).astype(np.float32) * 0.125
    part = np.ascontiguousarray(part.astype(np.float32))
    committed = splits * 32 - active
    for row in range(m):
        ob = np.full(D, 0xA5A5, dtype=np.uint16)
        of = np.zeros(D, dtype=np.float32)
        L.ko_attention_reduce_row(G, D, 8, ko.ptr(part), ko.ptr(stats), committed, active, splits, 0,
                                  row, ko.ptr(ob), ko.ptr(of))
        if row // G >= active:
            assert not ob.any()
            continue
        w = np.exp(mx[:, row].astype(np.float64) - mx[:, row].max())
        want = (w[:, None] * part[:, row]).sum(0) / (w * sm[:, row]).sum()
        got = ko.bf16_to_f32(ob).astype(np.float64)
        assert np.all(np.abs(got - want) <= np.abs(want) * 0.004 + 2e-6)


@pytest.mark.parametrize("fmt", [ko.INT4, ko.FP8])
def test_rounding_flips_turn_only_weights_on_a_boundary(fmt):
    """The GPU checks' allowance machinery (ko.rounding_flip_rows): with no slack nothing is
    turned; with a slack of a whole place every one of the heaviest tokens is, one at a time
    and together; a turned rounding moves the row by that token's share of a place, no more;
    and the untouched call still gives the plain tile."""
    committed, active, capacity, splits, head = 300, 8, 8, 3, 2
    store, pages, table = build_history(fmt, committed, active, seed=77)
    q = random_queries(capacity, 32, 78)
    tile_q = q[head, :capacity].reshape(capacity * G, D)
    kv = store.layer(1)
    base, base32 = ko.attention_tile_rows(fmt, H, G, D, tile_q, table, kv, head, committed, active,
                                          splits, capacity)
    fused_row = 3 * G + 1
    args = (fmt, H, G, D, tile_q, table, kv, head, committed, active, splits, capacity, fused_row)
    assert list(ko.rounding_flip_rows(*args, slack=0.0)) == []
    rows = list(ko.rounding_flip_rows(*args, top=3, slack=1.0, together=3))
    assert len(rows) == 7 and sorted(size for _, size, _ in rows) == [1, 1, 1, 2, 2, 2, 3]
    value = lambda bits: ko.bf16_to_f32(bits).astype(np.float64)
    for tokens, size, bits in rows:
        moved = np.linalg.norm(value(bits) - value(base[fused_row])) / np.linalg.norm(value(base[fused_row]))
        # one place of the weight's format, times at most the whole row
        assert 0 < moved <= size * (2.0 ** -7 if fmt != ko.FP8 else 2.0 ** -9) + 2e-3
    # at the real slack (twice the measured score deviation of the format's kernels) a minority
    # of bf16 weights is that close to a boundary (the window is 7.4e-4 wide, a place 3.9e-3 to
    # 7.8e-3); an fp16 place, 4.9e-4 to 9.8e-4, is no wider than the window, so on fp8 pages
    # most weights are; at a hundredth of the slack hardly any, in either format
    def near(slack):
        return sum(sum(1 for _, size, _ in ko.rounding_flip_rows(*args[:-1], r, top=6, slack=slack)
                       if size == 1) for r in range(0, 8 * G, 2))
    considered = 6 * 4 * G
    if fmt == ko.FP8:
        assert near(ko.flip_slack(fmt)) >= 0.5 * considered and near(ko.flip_slack(fmt) / 100) <= 6
    else:
        assert near(ko.flip_slack(fmt)) <= 0.4 * considered and near(ko.flip_slack(fmt) / 100) <= 2
    again, _ = ko.attention_tile_rows(fmt, H, G, D, tile_q, table, kv, head, committed, active,
                                      splits, capacity)
    assert np.array_equal(again, base)
    # the question belongs to the calling thread; the tile's worker threads must answer it too
    before = ko.lib().ko_threads()
    try:
        ko.set_threads(4)
        threaded = list(ko.rounding_flip_rows(*args, top=3, slack=1.0, together=3))
        spread, _ = ko.attention_tile_rows(fmt, H, G, D, tile_q, table, kv, head, committed, active,
                                           splits, capacity)
    finally:
        ko.set_threads(before)
    assert np.array_equal(spread, base)
    assert [(t, s) for t, s, _ in threaded] == [(t, s) for t, s, _ in rows]
    assert all(np.array_equal(a[2], b[2]) for a, b in zip(threaded, rows))
    store.close()
