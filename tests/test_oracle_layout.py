"""Oracle layout/addressing/planning against the reference's known answers.

Known answers are the reference's own (dev/tests/engine/q8_paged_kv_test.cc:17-75,
dev/tests/engine/paged_attention_plan_test.mm:104-176,
dev/tests/engine/q8_chunked_prefill_metal_test.mm:864-896,
dev/tests/engine/q8_flash_attention_metal_test.mm:53-56) and, where oracle/_ref
was built, the reference's real header code on random inputs.
"""
import ctypes as C
import itertools
import random

import numpy as np
import pytest

from oracle import kvoracle as ko

L = ko.lib()


def layout(layers, heads, dim, fmt=ko.INT8):
    return ko.Layout(layers, heads, dim, fmt, 0.0)


def geo(l):
    r = C.byref(l)
    return dict(model=L.ko_bytes_per_model_page(r), align=L.ko_extent_alignment_pages(r),
                lo=L.ko_minimum_extent_pages(r), hi=L.ko_maximum_extent_pages(r),
                data=L.ko_data_bytes_per_layer_page(r), scale=L.ko_scale_bytes_per_layer_page(r))


def test_byte_accounting_known_answers():
    bf16 = layout(16, 4, 256, ko.BF16)
    g = geo(bf16)
    assert g["model"] == 2_097_152 and g["align"] == 1 and (g["lo"], g["hi"]) == (32, 96)
    assert g["scale"] == 0 and 4096 * g["model"] == 8 * 1024 ** 3
    compact = layout(10, 2, 256, ko.BF16)
    g = geo(compact)
    assert g["model"] == 655_360 and g["align"] == 2 and (g["lo"], g["hi"]) == (104, 306)
    q8 = layout(16, 4, 256, ko.INT8)
    g = geo(q8)
    assert g["model"] == 1_064_960 == 2 * (512 + 8) * 1024
    assert g["align"] == 128 and (g["lo"], g["hi"]) == (128, 128)
    assert 16 * g["data"] == 512 * 1024 and 16 * g["scale"] == 8 * 1024
    assert 4608 * g["model"] == 4_907_335_680
    pf = lambda l, n: L.ko_extent_pages_for(C.byref(l), n)
    assert (pf(q8, 127), pf(q8, 128), pf(q8, 1000)) == (0, 128, 128)
    ci8 = layout(10, 2, 256, ko.INT8)
    g = geo(ci8)
    assert g["model"] == 332_800 and g["align"] == 256 and (g["lo"], g["hi"]) == (256, 512)
    assert (pf(ci8, 255), pf(ci8, 511), pf(ci8, 10_240), pf(ci8, 10_496)) == (0, 256, 512, 256)
    assert (pf(bf16, 31), pf(bf16, 448), pf(bf16, 97)) == (0, 64, 48)
    assert not L.ko_layout_valid(C.byref(ko.Layout(16, 4, 256, 0, 0.0)))
    # benchmark geometry: int4 = 1056 B/token/layer, fp8 = int8 geometry.
    i4 = layout(16, 4, 256, ko.INT4)
    assert geo(i4)["model"] == 540_672 == 16 * 32 * 1056 and geo(i4)["align"] == 128
    assert geo(layout(16, 4, 256, ko.FP8))["model"] == 1_064_960


def test_element_indices_known_answers():
    D, H, P = 256, 4, 32
    ke, ve = L.ko_key_element, L.ko_value_element
    assert ke(0, 0, 1, D) == ke(0, 0, 0, D) + 1
    assert ke(0, 1, 0, D) == ke(0, 0, 0, D) + D
    assert ve(0, 1, 0, D) == ve(0, 0, 0, D) + 1
    assert ve(0, 0, 1, D) == ve(0, 0, 0, D) + P
    assert ke(H - 1, P - 1, D - 1, D) == H * P * D - 1
    assert ve(H - 1, P - 1, D - 1, D) == H * P * D - 1


@pytest.mark.parametrize("heads,dim", [(4, 256), (2, 128), (8, 64)])
def test_element_indices_are_bijections(heads, dim):
    idx = np.array([[L.ko_key_element(h, t, d, dim), L.ko_value_element(h, t, d, dim)]
                    for h in range(heads) for t in range(32) for d in range(0, dim, 7)])
    full_k = {L.ko_key_element(h, t, d, dim) for h in range(heads) for t in range(32)
              for d in range(dim)} if dim == 64 else None
    assert idx.max() < heads * 32 * dim
    assert len(set(idx[:, 0])) == len(idx) and len(set(idx[:, 1])) == len(idx)
    if full_k is not None:
        assert full_k == set(range(heads * 32 * dim))
    assert sorted(L.ko_scale_element(h, t) for h in range(heads) for t in range(32)) == \
        list(range(heads * 32))


@pytest.mark.parametrize("fmt", [ko.INT8, ko.BF16, ko.INT4, ko.FP8])
def test_regions_tile_the_extent_without_gaps(fmt):
    # As dev/tests/engine/q8_page_storage_test.mm:54-76: every (layer, tensor,
    # page) span is distinct, in range and together they cover the extent.
    l = layout(3, 4, 256, fmt)
    db, sb = L.ko_data_bytes_per_layer_page(C.byref(l)), L.ko_scale_bytes_per_layer_page(C.byref(l))
    ep = 5
    spans = []
    for layer, tensor, index in itertools.product(range(3), range(4), range(ep)):
        size = sb if tensor % 2 else db
        if size:
            spans.append((L.ko_kv_offset(ep, db, sb, layer, tensor, index), size))
    spans.sort()
    assert spans[0][0] == 0
    for (a, n), (b, _) in zip(spans, spans[1:]):
        assert a + n == b
    assert spans[-1][0] + spans[-1][1] == ep * L.ko_bytes_per_model_page(C.byref(l))
    lay = L.ko_kv_layer_of(ep, db, sb, 2)
    assert lay.extent_pages == ep and lay.offset == 2 * ep * 2 * (db + sb)
    assert L.ko_page_entry(0x7F0000004000, 37) == 0x7F0000004000 | 37


def test_split_rules_known_answers():
    assert [L.ko_verify_splits(h, 8) for h in (0, 16384, 131072)] == [32, 33, 128]
    assert L.ko_verify_splits(31, 8) == 32
    for rows in range(1, 2049):
        tiles = (rows + 7) // 8
        assert L.ko_prefill_tiles(rows) == tiles
        assert L.ko_prefill_splits(tiles) == min(max(32 // tiles, 1), 32)
        pb, sb = C.c_uint64(), C.c_uint64()
        L.ko_prefill_workspace(rows, 24, 4, 256, C.byref(pb), C.byref(sb))
        fused = tiles * L.ko_prefill_splits(tiles) * 8 * 24
        assert (pb.value, sb.value) == (fused * 256 * 4, fused * 2 * 4)
        bp, bs = C.c_uint64(), C.c_uint64()
        L.ko_prefill_workspace_bound(rows, 24, 256, C.byref(bp), C.byref(bs))
        assert bp.value >= pb.value and bs.value >= sb.value
    for lanes in range(1, 5):
        pb, sb = C.c_uint64(), C.c_uint64()
        L.ko_verify_workspace(lanes, 8, 24, 256, C.byref(pb), C.byref(sb))
        fused = lanes * 8 * 128 * 24
        assert (pb.value, sb.value) == (fused * 256 * 4, fused * 2 * 4)


def test_chunk_validation_known_answers():
    p = ko.ChunkParams(129, 8, 32, 5)
    assert L.ko_chunk_validation(C.byref(p)) == 0 and L.ko_chunk_required_pages(C.byref(p)) == 5
    p.page_table_entries = 4
    assert L.ko_chunk_validation(C.byref(p)) == 4
    final = ko.ChunkParams(262144 - 1, 8, 32, (262159 + 31) // 32)
    assert L.ko_chunk_validation(C.byref(final)) == 0
    final.committed_tokens = 262159 - 8 + 1
    assert L.ko_chunk_validation(C.byref(final)) == 2
    assert L.ko_chunk_validation(C.byref(ko.ChunkParams(0, 0, 32, 1))) == 1
    assert L.ko_chunk_validation(C.byref(ko.ChunkParams(0, 2049, 2080, 99))) == 1
    assert L.ko_chunk_validation(C.byref(ko.ChunkParams(0, 8, 31, 1))) == 3
    assert C.sizeof(ko.ChunkParams) == 24 and C.sizeof(ko.PrefillParams) == 32
    assert C.sizeof(ko.VerifyParams) == 36 and C.sizeof(ko.KvLayer) == 8
    assert ko.PrefillParams.split_count.offset == 24 and ko.PrefillParams.score_scale.offset == 28
    assert ko.PrefillParams.kv.offset == 16


needs_ref = pytest.mark.skipif(ko.ref() is None, reason="oracle/_ref not built")


@needs_ref
def test_layout_matches_reference_headers():
    R = ko.ref()
    rng = random.Random(7)
    cases = [(16, 4, 256), (10, 2, 256), (1, 8, 64), (28, 2, 128), (40, 8, 128), (3, 1, 64)]
    for layers, heads, dim in cases:
        for fmt in (ko.INT8, ko.BF16, ko.INT4, ko.FP8):
            l = layout(layers, heads, dim, fmt)
            out = (C.c_uint64 * 8)()
            R.ref_layout(layers, heads, dim, fmt, out)
            g = geo(l)
            assert list(out)[:6] == [g["data"], g["scale"], g["model"], g["align"], g["lo"], g["hi"]]
            assert out[7] == L.ko_elements_per_layer_page(C.byref(l))
            for _ in range(40):
                n = rng.choice([rng.randrange(0, 600), rng.randrange(0, 40000)])
                assert L.ko_extent_pages_for(C.byref(l), n) == \
                    R.ref_extent_pages_for(layers, heads, dim, fmt, n)
            db, sb = g["data"], g["scale"]
            for _ in range(60):
                ep, layer = rng.randrange(1, 9000), rng.randrange(0, layers)
                tensor, index = rng.randrange(0, 4), rng.randrange(0, 9000)
                if ep * 2 * (db + sb) * layers >= 2 ** 32:
                    continue
                assert L.ko_kv_offset(ep, db, sb, layer, tensor, index) == \
                    R.ref_kv_offset(ep, db, sb, layer, tensor, index)
                lay = L.ko_kv_layer_of(ep, db, sb, layer)
                assert (lay.offset << 32) | lay.extent_pages == R.ref_kv_layer(ep, db, sb, layer)
    for _ in range(2000):
        h, t, d, dim = rng.randrange(8), rng.randrange(32), rng.randrange(64), rng.choice([64, 128, 256])
        assert L.ko_key_element(h, t, d, dim) == R.ref_key_element(h, t, d, dim)
        assert L.ko_value_element(h, t, d, dim) == R.ref_value_element(h, t, d, dim)
        assert L.ko_scale_element(h, t) == R.ref_scale_element(h, t)
    assert [R.ref_param_sizes(i) for i in range(4)] == [24, 32, 36, 8]


@needs_ref
def test_planning_matches_reference_headers():
    R = ko.ref()
    rng = random.Random(11)
    for _ in range(4000):
        committed = rng.choice([rng.randrange(0, 4096), rng.randrange(0, 262159)])
        rows = rng.choice([1, 8, 15, 16])
        assert L.ko_verify_splits(committed, rows) == R.ref_verify_splits(committed, rows)
        tokens = rng.choice([0, 1, 7, 8, 15, 2048, 2049, rng.randrange(0, 2100)])
        stride = rng.choice([0, 31, 32, 64, 2048, 2080, (tokens + 31) // 32 * 32])
        entries = rng.choice([0, (committed + tokens + 31) // 32, (committed + tokens + 31) // 32 - 1,
                              9000])
        entries = max(entries, 0)
        p = ko.ChunkParams(committed, tokens, stride, entries)
        assert L.ko_chunk_validation(C.byref(p)) == R.ref_chunk_validation(committed, tokens, stride, entries)
        assert L.ko_chunk_required_pages(C.byref(p)) == R.ref_chunk_required_pages(committed, tokens)
    for rows in range(1, 2049):
        assert L.ko_prefill_tiles(rows) == R.ref_prefill_tiles(rows)
