"""Oracle quantize-on-append: reference quantizer, reference patterns, invariants.

int8 and fp8 rows are compared bit for bit with the reference's own page
quantizers (dev/tests/engine/Q8PageFormatReference.hpp:141-180,
Fp8PageFormatReference.hpp:147-186) through oracle/_ref on the reference test's
sin/cos inputs (dev/tests/engine/q8_paged_kv_test.cc:92-110) and on random rows;
int4 shares that code path with qmax 7 and is pinned by invariants and an
independent numpy unpack; bf16 keeps the twelve edge bit patterns of
dev/tests/engine/paged_attention_plan_test.mm:681-699.
"""
import ctypes as C

import numpy as np
import pytest

from oracle import kvoracle as ko
import kvtestlib as T

L = ko.lib()
needs_ref = pytest.mark.skipif(ko.ref() is None, reason="oracle/_ref not built")
H, D = 4, 256


def append_rows(fmt, keys, values, committed=0, layers=2, layer=1, one_extent=False, seed=5):
    """Stores logical [H][T][D] fp32 rows at `committed`; returns (store, pages)."""
    tokens = keys.shape[1]
    n_pages = (committed + tokens + 31) // 32
    store = T.make_store(fmt, H, D, layers, n_pages, one_extent)
    pages = T.mixed_pages(store.extent_pages, store.page_count // store.extent_pages, n_pages, seed)
    table = store.entries(pages)
    stride = (tokens + 31) // 32 * 32
    ck, cv = T.chunk_buffers(keys, values, stride)
    p = ko.ChunkParams(committed, tokens, stride, n_pages, store.layer(layer))
    assert ko.store_chunk(fmt, H, D, ck, cv, table, p) == 1
    return store, pages


def sincos_inputs(tokens):
    t, h, d = np.meshgrid(np.arange(tokens), np.arange(H), np.arange(D), indexing="ij")
    keys = (2.5 * np.sin((t * 17 + h * 31 + d).astype(np.float32) * np.float32(0.013))).astype(np.float32)
    values = (1.75 * np.cos((t * 29 + h * 11 + d).astype(np.float32) * np.float32(0.017))).astype(np.float32)
    return keys, values  # [token][head][d]


@needs_ref
@pytest.mark.parametrize("tokens", [32, 17])
@pytest.mark.parametrize("fmt", [ko.INT8, ko.FP8])
def test_quantized_page_matches_reference_quantizer(fmt, tokens):
    R = ko.ref()
    rng = np.random.default_rng(tokens)
    for case in range(3):
        if case == 0:
            k, v = sincos_inputs(tokens)
        else:
            k = (rng.standard_normal((tokens, H, D)) * rng.choice([1e-3, 1.0, 300.0])).astype(np.float32)
            v = rng.standard_normal((tokens, H, D)).astype(np.float32)
            v[:, :, 5] *= 20
            k[0, 1, :] = 0.0  # a zero row: scale 0, codes 0
        kb, vb = ko.bf16_to_f32(ko.f32_to_bf16(k)), ko.bf16_to_f32(ko.f32_to_bf16(v))
        page = np.zeros(R.ref_q8_page_bytes(), dtype=np.uint8)
        fn = R.ref_quantize_q8_page if fmt == ko.INT8 else R.ref_quantize_fp8_page
        assert fn(ko.ptr(np.ascontiguousarray(kb)), ko.ptr(np.ascontiguousarray(vb)), tokens, ko.ptr(page)) == 0
        store, pages = append_rows(fmt, kb.transpose(1, 0, 2), vb.transpose(1, 0, 2), layers=1, layer=0)
        got = np.concatenate(T.slab_views(store, 0, int(pages[0])))
        assert np.array_equal(got, page)


@pytest.mark.parametrize("fmt,qmax", [(ko.INT8, 127), (ko.INT4, 7)])
@pytest.mark.parametrize("committed,tokens", [(0, 32), (33, 7), (129, 8), (31, 70)])
def test_integer_rows_invariants(fmt, qmax, committed, tokens):
    rng = np.random.default_rng(committed * 100 + tokens)
    k = rng.standard_normal((H, tokens, D)).astype(np.float32)
    v = rng.standard_normal((H, tokens, D)).astype(np.float32)
    k[:, :, [3, 77, 130, 255]] *= 20  # outlier channels
    k[1, 0, :] = 0
    store, pages = append_rows(fmt, k, v, committed)
    kb = ko.bf16_to_f32(ko.f32_to_bf16(k)).reshape(k.shape)
    vb = ko.bf16_to_f32(ko.f32_to_bf16(v)).reshape(v.shape)
    for t in range(tokens):
        logical = committed + t
        kc, ks, vc, vs = T.page_codes(store, 1, int(pages[logical // 32]))
        slot = logical % 32
        for src, codes, scales in ((kb, kc, ks), (vb, vc, vs)):
            for h in range(H):
                row, code, scale = src[h, t], codes[h, slot], scales[h, slot]
                m = np.abs(row).max()
                assert scale == (np.float32(m) / np.float32(qmax) if m else 0)
                assert np.abs(code).max() == (qmax if m else 0) and np.abs(code).max() <= qmax
                assert np.all(np.abs(code * scale - row) <= 0.51 * scale + 1e-7)  # q8_paged_kv_test.cc:123-126
                # the expected code, in numpy fp32 with the reference's operation order
                want = np.clip(np.rint(row * np.float32(qmax) / np.float32(m)), -qmax, qmax) if m else 0 * row
                assert np.array_equal(code, want)
    # slots before `committed` and other layers were never touched
    for page in set(int(p) for p in pages):
        assert not np.concatenate(T.slab_views(store, 0, page)).any()
    first = T.page_codes(store, 1, int(pages[0]))
    assert not first[0][:, :committed % 32 if committed < 32 else 32].any() or committed >= 32


def test_int4_expected_bytes_of_reference_plan_test():
    # dev/tests/engine/paged_attention_plan_test.mm:573-627 builds expected
    # bytes from chunk patterns (:409-417); byte = (code[d]&0xF)|(code[d+1]&0xF)<<4
    # at [head][token][d/2] for both tensors.
    rows, committed = 33, 31
    r, h, d = np.meshgrid(np.arange(rows), np.arange(H), np.arange(D), indexing="ij")
    k = (((r * 37 + h * 101 + d * 17) % 255 - 127).astype(np.float32) * np.float32(0.006))
    v = (((r * 53 + h * 79 + d * 29) % 255 - 127).astype(np.float32) * np.float32(0.007))
    store, pages = append_rows(ko.INT4, k.transpose(1, 0, 2), v.transpose(1, 0, 2), committed)
    for tensor, src in ((ko.KEYS, k), (ko.VALUES, v)):
        srcb = ko.bf16_to_f32(ko.f32_to_bf16(src)).reshape(src.shape)
        for row in range(rows):
            tok = committed + row
            views = T.slab_views(store, 1, int(pages[tok // 32]))
            for head in range(H):
                x = srcb[row, head]
                m = np.abs(x).max()
                code = np.clip(np.rint(x * np.float32(7.0) / m), -7, 7).astype(np.int32)
                want = ((code[0::2] & 0xF) | ((code[1::2] & 0xF) << 4)).astype(np.uint8)
                base = (head * 32 + tok % 32) * D // 2
                assert np.array_equal(views[tensor][base:base + D // 2], want)
                scale = views[tensor + 1].view(np.float32)[head * 32 + tok % 32]
                assert scale == np.float32(m) / np.float32(7.0)


def test_int8_rows_of_reference_prefill_test_patterns():
    # dev/tests/engine/q8_chunked_prefill_metal_test.mm:471-520: codes equal, scale
    # within 2e-7 of absmax/127 on keyPattern/valuePattern rows stored at 133.
    committed, tokens = 133, 32
    t, h, d = np.meshgrid(np.arange(tokens), np.arange(H), np.arange(D), indexing="ij")
    k = T.key_pattern(committed + t, h, d, 1).astype(np.float32)
    v = T.value_pattern(committed + t, h, d, 1).astype(np.float32)
    store, pages = append_rows(ko.INT8, k.transpose(1, 0, 2), v.transpose(1, 0, 2), committed)
    for tok in (0, 1, 26, 27, 31):
        kc, ks, vc, vs = T.page_codes(store, 1, int(pages[(committed + tok) // 32]))
        slot = (committed + tok) % 32
        for src, codes, scales in ((k, kc, ks), (v, vc, vs)):
            x = ko.bf16_to_f32(ko.f32_to_bf16(src[tok, 0]))
            m = np.abs(x).max()
            want = np.clip(np.rint(x * np.float32(127.0) / m), -127, 127)
            assert np.array_equal(codes[0, slot], want)
            assert abs(scales[0, slot] - m / 127.0) <= 2e-7


def test_bf16_store_keeps_every_bit_pattern():
    bits = np.array([0, 0x8000, 1, 0x8001, 0x007f, 0x0080, 0x4960, 0x7f7f, 0xff7f, 0x7f80, 0xff80,
                     0x7fc3], dtype=np.uint16)
    rows, committed = 33, 31
    stride = 64
    ck = bits[np.arange(H * stride * D) % 12].reshape(H, stride, D)
    cv = bits[(np.arange(H * D * stride) + 5) % 12].reshape(H, D, stride)
    n_pages = 2
    store = T.make_store(ko.BF16, H, D, 2, n_pages)
    pages = T.mixed_pages(store.extent_pages, store.page_count // store.extent_pages, n_pages, 1)
    p = ko.ChunkParams(committed, rows, stride, n_pages, store.layer(1))
    assert ko.store_chunk(ko.BF16, H, D, ck, cv, store.entries(pages), p) == 1
    for row in range(rows):
        tok = committed + row
        k, ks, v, vs = T.slab_views(store, 1, int(pages[tok // 32]))
        assert ks.size == 0 and vs.size == 0
        kk = k.view(np.uint16).reshape(H, 32, D)
        vv = v.view(np.uint16).reshape(H, D, 32)
        assert np.array_equal(kk[:, tok % 32, :], ck[:, row, :])
        assert np.array_equal(vv[:, :, tok % 32], cv[:, :, row])


@pytest.mark.parametrize("bad", ["tokens0", "stride", "short_table", "extent0", "context"])
def test_invalid_contract_writes_nothing(bad):
    # common/paged_store_row.h:14-29: an invalid lane returns without writes
    store = T.make_store(ko.INT8, H, D, 1, 4)
    pages = T.mixed_pages(store.extent_pages, store.page_count // store.extent_pages, 4, 2)
    for e in range(store.page_count // store.extent_pages):
        store.extent(e)[:] = 0xA5
    ck = np.full((H, 32, D), 0x3F80, dtype=np.uint16)
    p = ko.ChunkParams(40, 8, 32, 4, store.layer(0))
    if bad == "tokens0":
        p.chunk_tokens = 0
    elif bad == "stride":
        p.chunk_stride = 24
    elif bad == "short_table":
        p.page_table_entries = 1
    elif bad == "extent0":
        p.kv.extent_pages = 0
    else:
        p.committed_tokens = 262159 - 3
        p.page_table_entries = 9000
    assert ko.store_chunk(ko.INT8, H, D, ck, ck.reshape(H, D, 32), store.entries(pages), p) == 0
    for e in range(store.page_count // store.extent_pages):
        assert (store.extent(e) == 0xA5).all()


def test_verify_store_lanes_and_limits():
    # decode/paged_attention_store.metal:3-45: per-lane tables, rows <= 15, stride 32
    rng = np.random.default_rng(9)
    lanes = 3
    committed = [0, 31, 1023]
    counts = [(c + 8 + 31) // 32 for c in committed]
    store = T.make_store(ko.INT4, H, D, 2, sum(counts))
    ids = T.mixed_pages(store.extent_pages, store.page_count // store.extent_pages, sum(counts), 3)
    tables, first = [], 0
    for n in counts:
        tables.append(store.entries(ids[first:first + n]))
        first += n
    ck = ko.f32_to_bf16(rng.standard_normal((lanes, H, 32, D)).astype(np.float32)).reshape(lanes, H, 32, D)
    cv = ko.f32_to_bf16(rng.standard_normal((lanes, H, D, 32)).astype(np.float32)).reshape(lanes, H, D, 32)
    params = [ko.ChunkParams(committed[i], 8, 32, counts[i], store.layer(1)) for i in range(lanes)]
    params[1].chunk_tokens = 16  # over the verify row bound: this lane writes nothing
    assert ko.store_verify(ko.INT4, H, D, ck, cv, tables, params) == 2
    single = T.make_store(ko.INT4, H, D, 2, sum(counts))
    for lane in (0, 2):
        t = single.entries(ids[sum(counts[:lane]):sum(counts[:lane + 1])])
        assert ko.store_chunk(ko.INT4, H, D, ck[lane], cv[lane], t, params[lane]) == 1
    for e in range(store.page_count // store.extent_pages):
        assert np.array_equal(store.extent(e), single.extent(e))
