"""The C ABI loads without a GPU, exports every symbol include/kvx.h declares,
and its host-side rules agree with the oracle (no device calls here)."""
import ctypes as C
import os
import random
import re

import pytest

from oracle import kvoracle as ko
from richengine_amd import kvx

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    """The entries of the drop-in boundary (include/kvx.h) and the measurement and test hooks
    beside it (include/kvx_debug.h)."""
    names = set()
    for header in ("kvx.h", "kvx_debug.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(kvx?_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_debug_hooks_stay_out_of_the_boundary_header():
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "kvx.h")).read(), flags=re.S)
    assert "kvx_debug" not in text and "kvx_calibrate" not in text


def test_library_exports_every_declared_symbol():
    L = kvx.lib()
    names = declared_symbols()
    assert len(names) >= 50
    for name in names:
        assert hasattr(L, name), f"{name} is declared in include/kvx*.h but not exported"
    assert sorted(kvx.SYMBOLS) == names


def test_struct_layouts_match_the_reference_abi():
    assert C.sizeof(kvx.ChunkParams) == 24 and C.sizeof(kvx.PrefillParams) == 32
    assert C.sizeof(kvx.VerifyParams) == 36 and C.sizeof(kvx.KvLayer) == 8
    assert kvx.PrefillParams.kv.offset == 16 and kvx.PrefillParams.split_count.offset == 24
    assert kvx.VerifyParams.split_count.offset == 16 and kvx.VerifyParams.score_scale.offset == 32
    assert (kvx.INT8, kvx.BF16, kvx.INT4, kvx.FP8) == (1, 2, 3, 4)


def test_layout_rules_agree_with_the_oracle():
    L, O = kvx.lib(), ko.lib()
    rng = random.Random(5)
    for layers, heads, dim in [(16, 4, 256), (10, 2, 256), (1, 8, 64), (28, 2, 128), (40, 8, 128)]:
        for fmt in (1, 2, 3, 4):
            a, b = kvx.Layout(layers, heads, dim, fmt, 0.0), ko.Layout(layers, heads, dim, fmt, 0.0)
            ra, rb = C.byref(a), C.byref(b)
            assert L.kvx_layout_valid(ra) == O.ko_layout_valid(rb) == 1
            assert L.kvx_layout_data_bytes_per_layer_page(ra) == O.ko_data_bytes_per_layer_page(rb)
            assert L.kvx_layout_scale_bytes_per_layer_page(ra) == O.ko_scale_bytes_per_layer_page(rb)
            assert L.kvx_layout_bytes_per_layer_page(ra) == O.ko_bytes_per_layer_page(rb)
            assert L.kvx_layout_bytes_per_model_page(ra) == O.ko_bytes_per_model_page(rb)
            assert L.kvx_layout_extent_alignment_pages(ra) == O.ko_extent_alignment_pages(rb)
            assert L.kvx_layout_minimum_extent_pages(ra) == O.ko_minimum_extent_pages(rb)
            assert L.kvx_layout_maximum_extent_pages(ra) == O.ko_maximum_extent_pages(rb)
            for _ in range(50):
                n = rng.choice([rng.randrange(0, 700), rng.randrange(0, 50000)])
                assert L.kvx_layout_extent_pages_for(ra, n) == O.ko_extent_pages_for(rb, n)
            db, sb = O.ko_data_bytes_per_layer_page(rb), O.ko_scale_bytes_per_layer_page(rb)
            for _ in range(50):
                ep, layer, tensor, index = rng.randrange(1, 8000), rng.randrange(layers), rng.randrange(4), rng.randrange(8000)
                assert L.kvx_kv_offset(ep, db, sb, layer, tensor, index) == O.ko_kv_offset(ep, db, sb, layer, tensor, index)
            big = L.kvx_layout_largest_extent_pages(ra)
            assert big % L.kvx_layout_extent_alignment_pages(ra) == 0 and 0 < big <= 16383
            assert big * L.kvx_layout_bytes_per_model_page(ra) < 2 ** 32
    assert not L.kvx_layout_valid(C.byref(kvx.Layout(16, 4, 256, 0, 0.0)))
    assert not L.kvx_layout_valid(C.byref(kvx.Layout(0, 4, 256, 1, 0.0)))


def test_planning_rules_agree_with_the_oracle():
    L, O = kvx.lib(), ko.lib()
    rng = random.Random(6)
    assert [L.kvx_verify_splits(h, 8) for h in (0, 16384, 131072)] == [32, 33, 128]
    for _ in range(3000):
        committed, rows = rng.randrange(0, 262159), rng.choice([1, 8, 15, 16])
        assert L.kvx_verify_splits(committed, rows) == O.ko_verify_splits(committed, rows)
        pages = (committed + rows + 31) // 32
        assert L.kvx_decode_splits(committed, rows) == min(max(1, (pages + 31) // 32), 128)
        tokens = rng.choice([0, 1, 8, 2048, 2049, rng.randrange(0, 2100)])
        stride = rng.choice([0, 31, 32, 2048, 2080, (tokens + 31) // 32 * 32])
        entries = rng.choice([0, (committed + tokens + 31) // 32, max((committed + tokens + 31) // 32 - 1, 0), 9000])
        a, b = kvx.ChunkParams(committed, tokens, stride, entries), ko.ChunkParams(committed, tokens, stride, entries)
        assert L.kvx_chunk_validation(C.byref(a)) == O.ko_chunk_validation(C.byref(b))
    layout_a, layout_b = kvx.Layout(1, 4, 256, 3, 0.0), ko.Layout(1, 4, 256, 3, 0.0)
    for rows in range(1, 2049):
        assert L.kvx_prefill_splits(rows) == O.ko_prefill_splits(O.ko_prefill_tiles(rows))
        if rows % 37 and rows not in (1, 8, 9, 2048):
            continue
        pa, sa, pb, sb = C.c_uint64(), C.c_uint64(), C.c_uint64(), C.c_uint64()
        assert L.kvx_prefill_workspace(rows, 24, C.byref(layout_a), C.byref(pa), C.byref(sa)) == 0
        O.ko_prefill_workspace(rows, 24, 4, 256, C.byref(pb), C.byref(sb))
        assert (pa.value, sa.value) == (pb.value, sb.value)
        assert L.kvx_prefill_workspace_bound(rows, 24, C.byref(layout_a), C.byref(pa), C.byref(sa)) == 0
        O.ko_prefill_workspace_bound(rows, 24, 256, C.byref(pb), C.byref(sb))
        assert (pa.value, sa.value) == (pb.value, sb.value)
    for lanes in range(1, 5):
        pa, sa, pb, sb = C.c_uint64(), C.c_uint64(), C.c_uint64(), C.c_uint64()
        assert L.kvx_verify_workspace(lanes, 16, 24, C.byref(layout_a), C.byref(pa), C.byref(sa)) == 0
        O.ko_verify_workspace(lanes, 16, 24, 256, C.byref(pb), C.byref(sb))
        assert (pa.value, sa.value) == (pb.value, sb.value)
    # invalid geometry is refused with EINVAL and a message
    pa = C.c_uint64()
    assert L.kvx_prefill_workspace(0, 24, C.byref(layout_a), C.byref(pa), C.byref(pa)) == kvx.EINVAL
    assert L.kvx_prefill_workspace(2049, 24, C.byref(layout_a), C.byref(pa), C.byref(pa)) == kvx.EINVAL
    assert L.kvx_prefill_workspace(8, 25, C.byref(layout_a), C.byref(pa), C.byref(pa)) == kvx.EINVAL
    assert L.kvx_last_error()


def test_decode_and_verify_plans_size_the_launch_for_the_gpu():
    """kvx_decode_plan / kvx_verify_plan (no counterpart in the reference): every lane gets
    between 1 and the maximum number of splits, the partition covers its pages, and the launch
    has no more waves than the rule allows unless every split is already at its shortest."""
    import numpy as np
    rng = np.random.default_rng(3)
    H, QH = 4, 24
    pages = lambda tokens: (tokens + 31) // 32
    def decode_rule(committed, fmt, slots):
        """The rule for the lanes of one launch, restated."""
        lanes = len(committed)
        heads_pages = sum(pages(c + 1) for c in committed) * H
        small = heads_pages <= (4096 if fmt == kvx.INT4 else 2048) and max(pages(c + 1) for c in committed) <= 512
        per = max(-(-heads_pages // 1024), 4 if small else 8)
        if fmt == kvx.INT4:
            per = min(per, 32)
        while True:  # the first length whose waves fit the kernel's slots
            want = [min(max(1, -(-pages(c + 1) // per)), 512) for c in committed]
            if sum(want) * H <= slots or all(s == 1 for s in want):
                break
            per += 1
        if fmt == kvx.INT4 and sum(want) * H > 1024:
            # two waves on most SIMDs: long splits for exactly the first wave of every
            # SIMD, from the longest lane down while they fit, and splits of 0.58
            # of that length for the second waves; the least long length that fits
            counts = [pages(c + 1) for c in committed]
            order = sorted(range(lanes), key=lambda i: -counts[i])
            for longer in range(8, 8200):
                shorter = max(4, int(0.58 * longer))
                first = second = 0
                want = [0] * lanes
                for i in order:
                    as_long = -(-counts[i] // longer)
                    if first + as_long * H <= 1024:
                        want[i], first = as_long, first + as_long * H
                    else:
                        want[i] = -(-counts[i] // shorter)
                        second += want[i] * H
                if second <= 1024 and max(want) <= 512:
                    break
            assert first <= 1024 and second <= 1024
        return want

    def verify_rule(committed, rows, fmt):
        fused = rows * (QH // H)
        blocks = -(-fused // 32) if fused > 16 else 1
        if fmt != kvx.INT4 and 64 < fused <= 128:
            blocks = 4                             # waves of a workgroup that shares its pages
            if fmt == kvx.BF16 and fused <= 96:
                blocks = 2                         # two waves of 48 rows
        if fmt == kvx.INT4 and fused > 16 and 26 * -(-fused // 48) < 15 * -(-fused // 32):
            blocks = -(-fused // 48)  # the int4 kernel for 48 fused rows per wave
        counts = [pages(c + rows) for c in committed]
        # the int4 kernel for blocks of 32 rows of longer lanes: two waves per SIMD from 16 lanes on
        slots = 2048 if (fmt == kvx.INT4 and fused > 32 and blocks == -(-fused // 32)
                         and len(committed) >= 16) else 1024
        small = sum(counts) * H * blocks <= 2048 and max(counts) <= 512
        per = max(-(-sum(counts) * H * blocks // slots), 4 if small else 8)
        while True:  # the first length that fits one round of waves
            want = [min(max(1, -(-n // per)), 128) for n in counts]
            if sum(want) * H * blocks <= slots or all(s == 1 for s in want):
                break
            per += 1
        return want

    for trial in range(40):
        lanes = int(rng.integers(1, 100))   # past 32 lanes: several launches, each planned alone
        top = int(rng.choice([300, 4000, 70000]))
        committed = [int(x) for x in rng.integers(0, top, lanes)]
        groups = [committed[i:i + 32] for i in range(0, lanes, 32)]
        for fmt, slots in ((kvx.INT4, 2048), (kvx.INT8, 1024), (kvx.BF16, 1024), (kvx.FP8, 1024)):
            plan = kvx.decode_plan(committed, H, fmt)
            assert plan == sum((decode_rule(g, fmt, slots) for g in groups), [])
        for rows, fmt in ((2, kvx.INT4), (8, kvx.INT4), (8, kvx.INT8), (16, kvx.INT4), (16, kvx.BF16)):
            plan = kvx.verify_plan(committed, rows, H, QH, fmt)
            assert plan == sum((verify_rule(g, rows, fmt) for g in groups), [])
            counts = [pages(c + rows) for c in committed]
            assert all(1 <= s <= 128 and s <= max(n, 1) for s, n in zip(plan, counts))
    # by layout: head dimension 256 is the plan above; 128 and 64 plan one round of single waves
    import ctypes as C
    for heads, dim, fmt, want in ((4, 256, kvx.INT4, kvx.decode_plan([8191] * 32, 4, kvx.INT4)),
                                  (2, 128, kvx.INT4, [64] * 32),    # 256 pages x 2 heads x 32 lanes on 4096 waves: 4 pages a split
                                  (2, 128, kvx.FP8, [32] * 32),     # other than int4 at 128: 2048 waves, 8 pages a split
                                  (8, 64, kvx.INT8, [16] * 32),     # 256 x 8 x 32 on 4096: 16 pages a split
                                  (2, 128, kvx.BF16, [16] * 32)):    # bf16 pages: half the waves
        layout = kvx.Layout(1, heads, dim, fmt, 0.0)
        out = (C.c_uint32 * 32)()
        kvx.check(kvx.lib().kvx_decode_plan_for(C.byref(layout), (C.c_uint32 * 32)(*([8191] * 32)), 32, out))
        assert list(out) == want, (heads, dim, list(out)[:3])
    layout = kvx.Layout(1, 2, 128, kvx.INT4, 0.0)
    out = (C.c_uint32 * 2)()
    kvx.check(kvx.lib().kvx_decode_plan_for(C.byref(layout), (C.c_uint32 * 2)(0, 100000), 2, out))
    assert list(out) == [1, 128]                                  # at most 128 splits, at least 4 pages each
    assert kvx.lib().kvx_decode_plan_for(C.byref(layout), (C.c_uint32 * 1)(262144 + 15), 1, out) != 0
    # a small launch takes shorter splits: one sequence of 8192 tokens, 64 splits of 4 pages
    assert kvx.decode_plan([8191], H, kvx.INT4) == [64] and kvx.decode_plan([8191], H, kvx.INT8) == [64]
    assert kvx.decode_plan([8191] * 3, H, kvx.INT4) == [64] * 3 and kvx.decode_plan([8191] * 3, H, kvx.BF16) == [32] * 3
    assert kvx.decode_plan([32767], H, kvx.INT4) == [128]   # 256 splits would be too many to merge
    # chunked prefill: one split while the paired tiles fill half of the wave slots, else the
    # largest count whose one-tile lanes fit one round (and leave 8 pages per split)
    for fmt in (kvx.INT4, kvx.INT8, kvx.FP8, kvx.BF16):
        single_slots = 2048 if fmt == kvx.INT4 else 1024
        slots = 1024 if fmt == kvx.BF16 else 2048
        for committed, rows in ((16384, 64), (16384, 256), (16384, 512), (16384, 2048), (0, 256),
                                (100, 7), (3000, 264), (3004, 264), (16388, 512), (0, 1024), (2048, 1024),
                                (65536, 1024), (1024, 2048), (16388, 2048), (512, 768)):
            tiles = -(-rows // 8)
            paired = -(-tiles // 2) * H * -(-(16 * (QH // H)) // 32)
            want = 1
            width = 0
            if fmt != kvx.INT4 and rows >= 64:           # lanes of several tiles, a workgroup each
                fused = 8 * (QH // H)
                width = 4 if 4 * fused <= 192 else 2 if 2 * fused <= 192 else 0
                width = width if width * fused >= 96 else 0
            workgroups = -(-tiles // width) * H if width else 0
            alike = width and (committed % 32 == 0 if width == 4 else
                               (committed % 16 == 0 or committed % 16 >= 9))
            if width and 4 * workgroups >= 3 * 256:
                want = 1
            elif alike:
                want = max(1, min(-(-256 // workgroups), max(1, pages(committed + rows) // 8), 32))
            elif fmt == kvx.INT4 and 4 * paired >= single_slots:
                # equally long waves take the slots round by round: the fewest splits (of 16
                # pages of the average tile's history or more) whose rounds are nine tenths full
                pairable = committed % 16 == 0 or committed % 16 >= 9
                most = max(1, min(pages(committed + rows // 2) // 16, 32)) if pairable else 1
                room = lambda s: -(-paired * s // single_slots) * single_slots
                full = [s for s in range(1, most + 1) if 10 * paired * s >= 9 * room(s)]
                want = full[0] if full else max(range(1, most + 1), key=lambda s: (paired * s / room(s), -s))
            elif 2 * paired < single_slots:
                by_pages = max(1, pages(committed + rows) // 8)
                pairable = tiles >= 2 and (committed % 16 == 0 or committed % 16 >= 9)
                if fmt == kvx.INT4 and tiles < 64:
                    pairable = False
                together = max(1, min(single_slots // paired, by_pages, 32))
                if pairable and together >= 2 and 2 * paired * together >= single_slots:
                    want = together                                            # tiles stay paired
                else:
                    want = min(slots // (tiles * H * -(-(8 * (QH // H)) // 16)), by_pages, 32)
                    want = want if want >= 2 else 1
            assert kvx.prefill_plan(committed, rows, H, QH, fmt) == want
    assert kvx.prefill_plan(16384, 256, H, QH, kvx.INT4) == 5      # 384 waves of single tiles per split
    assert kvx.prefill_plan(16384, 256, H, QH, kvx.BF16) == 8      # 32 workgroups of four tiles each
    assert kvx.prefill_plan(16384, 1024, H, QH, kvx.FP8) == 2      # 128 workgroups
    assert kvx.prefill_plan(16384, 2048, H, QH, kvx.INT8) == 1     # 256 workgroups
    assert kvx.prefill_plan(16384, 1024, H, QH, kvx.INT4) == 5     # 768 waves of paired tiles: 3840 on 4096 slots
    assert kvx.prefill_plan(16388, 256, H, QH, kvx.BF16) == 2      # 384 of single tiles
    assert kvx.prefill_plan(16384, 2048, H, QH, kvx.INT4) == 4     # 1536 waves: three full rounds of 2048
    assert kvx.prefill_plan(0, 2048, H, QH, kvx.INT4) == 1         # 32 pages before the average tile: nothing to cut
    assert kvx.prefill_plan(0, 1024, H, QH, kvx.INT4) == 1
    assert kvx.prefill_plan(16384, 2048, H, QH, kvx.INT4, sequences=4) == 1   # 6144 waves already
    assert kvx.prefill_plan(16384, 2048, H, QH, kvx.INT4, sequences=2) == 2
    assert kvx.prefill_plan(16384, 256, H, QH, kvx.BF16, sequences=4) == 2    # 128 workgroups
    assert kvx.lib().kvx_prefill_plan_batch(16384, 256, H, QH, kvx.INT4, 0) == 0
    # contexts past the interface's maximum are refused before any planning; absurd head counts
    # neither divide by a wrapped zero nor walk the split lengths one by one for seconds
    import time
    for committed in ([262144 + 15], [5, 0xFFFFFFFF]):
        with pytest.raises(kvx.KvxError):
            kvx.decode_plan(committed, H, kvx.INT4)
        with pytest.raises(kvx.KvxError):
            kvx.verify_plan(committed, 16, H, QH, kvx.INT4)
    started = time.perf_counter()
    for fmt in (kvx.INT4, kvx.INT8, kvx.BF16):
        for heads in (748871255, 1 << 22, 0xFFFFFFFF):
            plan = kvx.decode_plan([262144, 32146, 6, 2048] * 8, heads, fmt)
            assert all(1 <= s <= 512 for s in plan)
            plan = kvx.verify_plan([262144, 32146, 6, 2048] * 8, 15, heads, heads, fmt)
            assert all(1 <= s <= 128 for s in plan)
    assert time.perf_counter() - started < 2.0
    # wave counts saturate: absurd shapes get some count in 1..32 instead of a wrapped division
    for fmt in (kvx.INT4, kvx.INT8, kvx.BF16):
        for heads, query_heads, sequences in ((1 << 31, 1 << 31, 1 << 31), (2, 1 << 31, 0xFFFFFFFF),
                                              (1 << 30, 3 << 30, 1 << 30), (4, 24, 0xFFFFFFFF)):
            for rows in (8, 2048, 0xFFFFFFFF):
                assert 1 <= kvx.lib().kvx_prefill_plan_batch(0xFFFFFFF0, rows, heads, query_heads, fmt,
                                                             sequences) <= 32
    with pytest.raises(kvx.KvxError):
        kvx.prefill_plan(16384, 256, 4, 6)
    assert kvx.verify_plan([65536] * 4, 16, H, QH) == [21] * 4          # three waves of 32 fused rows
    assert kvx.verify_plan([65536] * 4, 16, H, QH, kvx.BF16) == [32] * 4  # two waves of 48 rows that share their pages
    assert kvx.verify_plan([65536] * 4, 16, H, QH, kvx.INT8) == [16] * 4  # four waves that share their pages
    with pytest.raises(kvx.KvxError):
        kvx.verify_plan([10], 8, 4, 6)


def test_hot_kernels_stay_out_of_scratch_memory():
    """What the compiler reported when the library was built (written next to it by
    richengine_amd/build.py): the kernels of the decode path and the verify kernel must
    not touch scratch memory -- a spill reload or an argument block moved to scratch waits
    behind every page load in flight -- and the int4 decode kernel must fit two waves per
    SIMD."""
    import json
    import os
    from richengine_amd import build as kvx_build
    if not os.path.exists(kvx_build.RESOURCES):
        pytest.skip("the library was built without the compiler's resource report")
    report = json.load(open(kvx_build.RESOURCES))

    def one(fragment):
        names = [n for n in report if fragment in n]
        assert len(names) == 1, (fragment, names)
        return report[names[0]]

    for fragment in ("decode_int4_kernelE", "decode_int4_quad_kernel", "decode_int4_tiles_kernel", "verify_int4_kernel",
                     "verify32_int4_kernel", "verify48_int4_kernel", "prefill_int4_kernel",
                     "matrix_merge_kernelILj1E", "matrix_merge_kernelILj8E",   # one wave per row; ranged
                     "attend_wide_kernelILj1ELj1ELj2ELb0E",    # int8, one block, two waves per SIMD
                     "attend_wide_kernelILj4ELj1ELj2ELb0E",    # fp8
                     "attend_wide_kernelILj2ELj1ELj1ELb0E",    # bf16 decode
                     "attend_wide_kernelILj1ELj1ELj2ELb1E", "attend_wide_kernelILj4ELj1ELj2ELb1E",
                     "attend_wide_kernelILj2ELj1ELj1ELb1E",    # the same three for prefill tiles
                     "attend_wide_kernelILj1ELj2ELj1ELb0E", "attend_wide_kernelILj4ELj2ELj1ELb0E",
                     # the same two with page loads that may stay in the caches (prefill tiles)
                     "attend_wide_kernelILj1ELj2ELj1ELb1E", "attend_wide_kernelILj4ELj2ELj1ELb1E"):
        r = one(fragment)
        assert r["scratchsize"] == 0 and r["vgprs_spill"] == 0, (fragment, r)
    assert one("decode_int4_kernelE")["occupancy"] == 2 and one("decode_int4_quad_kernel")["occupancy"] == 2
    # two blocks over one page set: every accumulator in the first register file
    assert one("verify32_int4_kernel")["agprs"] == 0 and one("prefill_int4_kernel")["agprs"] == 0
    # the workgroup-shared prefill kernels (int8, bf16, fp8 pages; two and three row blocks
    # per wave): one wave per SIMD with all 512 registers; the byte formats' three-block forms
    # park a few set-up values in scratch memory, none of them touched inside the page loop
    # (no scratch access in the loop's assembly when this bound was set)
    # (the same kernels with loads that do not stay in the caches serve tree verify, and forms
    # with two waves and two LDS copies a chain of 8 rows)
    for fmt in (1, 2, 4):
        for blocks in (2, 3):
            for reused in ((0, 1) if blocks == 2 else (1,)):
                r = one(f"group_wide_kernelILj{fmt}ELj{blocks}ELj4ELb{reused}E")
                if fmt != 2 and blocks == 3:
                    assert r["vgprs_spill"] <= 10, (fmt, blocks, r)
                else:
                    assert r["scratchsize"] == 0 and r["vgprs_spill"] == 0, (fmt, blocks, r)
    for fmt in (1, 2, 4):
        r = one(f"group_wide_kernelILj{fmt}ELj2ELj2ELb0E")
        assert r["scratchsize"] == 0 and r["vgprs_spill"] == 0, r
    r = one("group_wide_kernelILj2ELj3ELj2ELb0E")      # bf16, two waves of 48 rows, direct loads
    assert r["scratchsize"] == 0 and r["vgprs_spill"] == 0, r
    # head dimensions 64 and 128, a wave per tile: no scratch, and two (128) or three and more
    # (64) waves per SIMD beside the staged copies
    for fmt in (1, 2, 3, 4):
        for dim, least in ((128, 2), (64, 3)):
            r = one(f"attend_split_small_wave_kernelILj{fmt}ELj{dim}E")
            assert r["scratchsize"] == 0 and r["vgprs_spill"] == 0 and r["occupancy"] >= least, (fmt, dim, r)
    # the same tiles shared by four waves (verify and prefill of more than 16 fused rows): the tile
    # is inlined into its kernels; called as a function it cost them 200 to 300 bytes of stack
    for kernel in ("attend_split_small_kernel", "prefill_split_small_kernel"):
        for fmt in (1, 2, 3, 4):
            for dim in (128, 64):
                for blocks in (1, 2):
                    r = one(f"{kernel}ILj{fmt}ELj{dim}ELj{blocks}E")
                    assert r["scratchsize"] == 0 and r["vgprs_spill"] == 0, (kernel, fmt, dim, blocks, r)
    # the kernels whose accumulators fill the second register file (48-row verify, two-block
    # bf16): since their rescaling names the accumulators there, nothing spills
    for fragment in ("verify48_int4_kernel", "attend_wide_kernelILj2ELj2ELj1ELb0E",
                     "attend_wide_kernelILj2ELj2ELj1ELb1E"):
        r = one(fragment)
        assert r["scratchsize"] == 0 and r["vgprs_spill"] == 0, (fragment, r)
    assert one("attend_wide_kernelILj1ELj1ELj2ELb0E")["occupancy"] == 2
    for fmt in (1, 2, 3, 4):
        assert one(f"13append_kernelILj{fmt}E")["scratchsize"] == 0
        assert one(f"prepare_append_kernelILj{fmt}E")["scratchsize"] == 0


def test_storage_refuses_geometry_the_kernels_cannot_index():
    """A page's bytes are indexed in 32 bits on the device: head counts whose page bytes would
    wrap are refused when the storage is made (with kv_heads = 2**19 + 4 the wrapped sizes are
    those of 4 heads), the layout functions answer in 64 bits, and a pool cannot have so many
    extents that its host tables alone take gigabytes."""
    import ctypes as C
    L = kvx.lib()
    wrapped = kvx.Layout(1, (1 << 19) + 4, 256, kvx.INT8, 0.0)
    L.kvx_layout_data_bytes_per_layer_page.restype = C.c_uint64
    assert L.kvx_layout_data_bytes_per_layer_page(C.byref(wrapped)) == 32 * ((1 << 19) + 4) * 256
    for heads, layers, pages, extent_pages in (((1 << 19) + 4, 1, 256, 128), (4097, 1, 256, 128),
                                               (4, 65537, 256, 128), (1, 1, 3 << 20, 1)):
        with pytest.raises(kvx.KvxError):
            kvx.Storage(layers, heads, 64, kvx.INT8, pages, extent_pages, accounting=True)
    kvx.Storage(1, 1, 64, kvx.INT8, 1 << 20, 1, accounting=True).close()


def test_prefill_groups_of_tiles_rule():
    """kvx_debug_prefill_tiles_together: groups only on a history that ends on a page boundary, only
    at head dimensions 64 and 128, as many tiles as keep four waves to a SIMD, and only in launches
    of enough workgroups (256 where a tile alone leaves waves idle, 1024 otherwise)."""
    import ctypes as C

    def together(heads, group, dim, committed, rows, splits, fmt=kvx.INT4):
        layout = kvx.Layout(1, heads, dim, fmt, 0.0)
        return kvx.lib().kvx_debug_prefill_tiles_together(C.byref(layout), heads * group, committed, rows, splits)

    assert together(8, 4, 64, 16384, 2048, 1) == 4          # 64 groups x 8 heads = 512 workgroups
    assert together(8, 4, 64, 16385, 2048, 1) == 1          # not on a page boundary
    assert together(8, 4, 64, 16384, 512, 1) == 1           # 128 workgroups
    assert together(8, 4, 64, 16384, 512, 2) == 4           # 256
    assert together(2, 8, 64, 16384, 2048, 2) == 1          # every wave has a block: 512 < 1024
    assert together(2, 8, 64, 16384, 2048, 4) == 2
    assert together(2, 8, 128, 16384, 2048, 8) == 1         # two blocks a wave at 128: never
    assert together(2, 4, 128, 16384, 2048, 1) == 2 and together(4, 2, 128, 16384, 2048, 1) == 4
    assert together(4, 6, 256, 16384, 2048, 4) == 1         # head dimension 256 has kernels of its own
    assert together(8, 4, 64, 0, 8, 32) == 1                # one tile
    assert together(8, 3, 64, 0, 8, 32) == 1 and together(8, 0, 64, 0, 8, 32) == 0


def test_prefill_plan_by_layout():
    """kvx_prefill_plan_for: head dimension 256 is kvx_prefill_plan_batch; 64 and 128 take the fewest
    splits that make 4096 workgroups (groups of tiles counted as the kernels form them), none
    shorter than 4 pages."""
    import ctypes as C

    def plan(heads, group, dim, committed, rows, sequences=1, fmt=kvx.INT4):
        layout = kvx.Layout(1, heads, dim, fmt, 0.0)
        return kvx.lib().kvx_prefill_plan_for(C.byref(layout), committed, rows, heads * group, sequences)

    assert plan(8, 4, 64, 16384, 2048) == 8         # 64 groups of four tiles x 8 heads x 8 splits
    assert plan(8, 4, 64, 16385, 2048) == 2         # tile by tile: 256 tiles x 8 heads x 2
    assert plan(2, 8, 128, 16384, 2048) == 8        # 256 tiles x 2 heads x 8
    assert plan(8, 4, 64, 8192, 256) == 32          # 8 groups x 8 heads: 32 splits are the most there are
    assert plan(2, 8, 128, 0, 64) == 1              # two pages of history: nothing to cut
    assert plan(2, 8, 128, 1000, 64) == 8           # 33 pages: at least 4 to a split
    for committed, rows, sequences in ((16384, 2048, 1), (16384, 2048, 4), (100, 256, 2)):
        assert plan(4, 6, 256, committed, rows, sequences) == kvx.prefill_plan(committed, rows, 4, 24, kvx.INT4, sequences)
    assert plan(8, 0, 64, 0, 8) == 0 and plan(8, 4, 64, 0, 8, sequences=0) == 0
    bad = kvx.Layout(1, 0, 64, kvx.INT4, 0.0)
    assert kvx.lib().kvx_prefill_plan_for(C.byref(bad), 0, 8, 8, 1) == 0
    # absurd sizes neither hang nor wrap
    for committed, rows in ((0xFFFFFFFF, 0xFFFFFFFF), (0, 0), (0xFFFFFFFF, 1), (5, 0xFFFFFFFF)):
        assert 0 <= plan(8, 4, 64, committed, rows) <= 32
