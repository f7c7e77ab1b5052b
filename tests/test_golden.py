"""Committed golden vectors (tests/golden/reference_vectors.npz, written by
tests/golden/make_vectors.py from the reference's own host code) against the
oracle, the library's host functions and, on the GPU, quantize-on-append.

Unlike the tests that call oracle/_ref directly, these run wherever the
repository is checked out: the expected values travel as data."""
import ctypes as C
import os

import numpy as np
import pytest

from oracle import kvoracle as ko
from richengine_amd import kvx
import kvtestlib as T

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.npz"))
L = ko.lib()
H, D = 4, 256


def layouts(make):
    for (layers, heads, dim, fmt), want in zip(G["layout_in"], G["layout_out"]):
        yield make(int(layers), int(heads), int(dim), int(fmt), 0.0), [int(x) for x in want]


def test_oracle_layout_numbers():
    for i, (l, want) in enumerate(layouts(ko.Layout)):
        r = C.byref(l)
        got = [L.ko_data_bytes_per_layer_page(r), L.ko_scale_bytes_per_layer_page(r),
               L.ko_bytes_per_model_page(r), L.ko_extent_alignment_pages(r),
               L.ko_minimum_extent_pages(r), L.ko_maximum_extent_pages(r),
               int(bool(L.ko_layout_valid(r))), L.ko_elements_per_layer_page(r)]
        if not want[6]:
            assert not got[6]
            continue
        assert got == want
        for pages, extent in zip(G["layout_extent_pages_in"], G["layout_extent_pages_out"][i]):
            assert L.ko_extent_pages_for(r, int(pages)) == int(extent)


def test_library_layout_numbers():
    K = kvx.lib()
    for i, (l, want) in enumerate(layouts(kvx.Layout)):
        r = C.byref(l)
        if not want[6]:
            assert not K.kvx_layout_valid(r)
            continue
        got = [K.kvx_layout_data_bytes_per_layer_page(r), K.kvx_layout_scale_bytes_per_layer_page(r),
               K.kvx_layout_bytes_per_model_page(r), K.kvx_layout_extent_alignment_pages(r),
               K.kvx_layout_minimum_extent_pages(r), K.kvx_layout_maximum_extent_pages(r)]
        assert got == want[:6] and K.kvx_layout_valid(r)
        for pages, extent in zip(G["layout_extent_pages_in"], G["layout_extent_pages_out"][i]):
            assert K.kvx_layout_extent_pages_for(r, int(pages)) == int(extent)


def test_offsets_and_element_indices():
    K = kvx.lib()
    for row, want in zip(G["offset_in"], G["offset_out"]):
        args = [int(x) for x in row]
        assert L.ko_kv_offset(*args) == int(want)
        assert K.kvx_kv_offset(*args) == int(want)
    for c, k, v, s in zip(G["element_in"], G["element_key"], G["element_value"], G["element_scale"]):
        c = [int(x) for x in c]
        assert L.ko_key_element(*c) == int(k) and L.ko_value_element(*c) == int(v)
        assert L.ko_scale_element(c[0], c[1]) == int(s)


def test_codecs():
    x = G["codec_in"]
    assert np.array_equal(ko.f32_to_bf16(x).ravel(), G["bf16_bits"])
    assert np.array_equal(np.array([L.ko_float_to_bf16(float(v)) for v in x], dtype=np.uint16),
                          G["bf16_bits"])
    assert np.array_equal(np.array([L.ko_float_to_fp8e4m3(float(v)) for v in x], dtype=np.uint8),
                          G["fp8_codes"])
    got = np.array([L.ko_fp8e4m3_to_float(c) for c in range(256)], dtype=np.float32)
    assert np.array_equal(got.view(np.uint32), G["fp8_decode"].view(np.uint32))
    staged = np.array([L.ko_round_to_f16(float(v)) for v in x], dtype=np.float32)
    assert np.array_equal(staged.view(np.uint32), G["stage_out"].view(np.uint32))


def test_planning():
    K = kvx.lib()
    for (committed, rows), want in zip(G["splits_in"], G["splits_out"]):
        assert L.ko_verify_splits(int(committed), int(rows)) == int(want)
        assert K.kvx_verify_splits(int(committed), int(rows)) == int(want)
    for rows, want in zip(G["tiles_in"], G["tiles_out"]):
        assert L.ko_prefill_tiles(int(rows)) == int(want)
    for c, error, pages in zip(G["chunk_in"], G["chunk_error"], G["chunk_pages"]):
        p = ko.ChunkParams(*[int(x) for x in c])
        assert L.ko_chunk_validation(C.byref(p)) == int(error)
        assert L.ko_chunk_required_pages(C.byref(p)) == int(pages)
        q = kvx.ChunkParams(*[int(x) for x in c])
        assert K.kvx_chunk_validation(C.byref(q)) == int(error)


def identity_cases():
    spans, first = G["identity_spans"], G["identity_spans_first"]
    for (which, begin, tokens), want in zip(G["identity_cases"], G["identity_out"]):
        mine = [tuple(int(w) for w in row) for row in spans[first[int(which)]:first[int(which) + 1]]]
        yield mine, int(begin), int(tokens), (int(want[0]), int(want[1]))


def test_image_identity_values_of_the_reference():
    """The 128-bit values of engine::blockImageIdentity (runtime/engine/cache/KvCache.cpp:29-52),
    written from the reference's own compiled function: the oracle's restatement and the
    library's entry give the same bits, for pages and for blocks that are no page, for spans
    before, inside, across and after the block, and for a span whose 32-bit end wraps."""
    from oracle import prefix_oracle as po
    seen_zero = seen_value = 0
    for spans, begin, tokens, want in identity_cases():
        assert po.block_image_identity(begin, tokens, spans) == want, (spans, begin, tokens)
        assert kvx.block_image_identity(begin, tokens, spans) == want, (spans, begin, tokens)
        seen_zero += want == (0, 0)
        seen_value += want != (0, 0)
    assert seen_zero > 50 and seen_value > 50


def test_image_identity_fixture_is_what_the_reference_returns():
    """Where the reference checkout was present at build time: the fixture against a fresh
    call of the reference's function."""
    if ko.ref_image_identity(0, 32, []) is None:
        pytest.skip("oracle/_ref/libkvref_cache.so was not built")
    for spans, begin, tokens, want in identity_cases():
        assert ko.ref_image_identity(begin, tokens, spans) == want


PAGES = [("q8", ko.INT8, "a"), ("q8", ko.INT8, "b"), ("f8", ko.FP8, "a"), ("f8", ko.FP8, "b")]


def golden_rows(name, case):
    """Logical [head][token][d] fp32 rows and the expected page bytes."""
    k = ko.bf16_to_f32(G[f"{name}_{case}_keys_bf16"]).reshape(G[f"{name}_{case}_keys_bf16"].shape)
    v = ko.bf16_to_f32(G[f"{name}_{case}_values_bf16"]).reshape(k.shape)
    return k.transpose(1, 0, 2), v.transpose(1, 0, 2), G[f"{name}_{case}_page"]


@pytest.mark.parametrize("name,fmt,case", PAGES)
def test_oracle_append_writes_the_reference_page(name, fmt, case):
    k, v, want = golden_rows(name, case)
    tokens = k.shape[1]
    store = T.make_store(fmt, H, D, 1, 1)
    pages = T.mixed_pages(store.extent_pages, store.page_count // store.extent_pages, 1, 3)
    ck, cv = T.chunk_buffers(k, v, 32)
    p = ko.ChunkParams(0, tokens, 32, 1, store.layer(0))
    assert ko.store_chunk(fmt, H, D, ck, cv, store.entries(pages), p) == 1
    assert np.array_equal(np.concatenate(T.slab_views(store, 0, int(pages[0]))), want)


@pytest.mark.gpu
@pytest.mark.parametrize("name,fmt,case", PAGES)
def test_gpu_append_writes_the_reference_page(name, fmt, case):
    import torch
    import gpulib as Gp
    k, v, want = golden_rows(name, case)
    tokens = k.shape[1]
    tw = Gp.Twin(fmt, H, D, 1, 1)
    pages = tw.pages(1, 3)
    _, td = tw.tables(pages)
    ck, cv = T.chunk_buffers(k, v, 32)
    kvx.append(tw.dev, 0, Gp.dev(ck), Gp.dev(cv), [td], [kvx.ChunkParams(0, tokens, 32, 1)], H * 32 * D)
    torch.cuda.synchronize()
    tw.download()
    assert np.array_equal(np.concatenate(T.slab_views(tw.host, 0, int(pages[0]))), want)
    tw.close()
