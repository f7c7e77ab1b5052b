"""Writes tests/golden/reference_vectors.npz from the reference's own host code.

Run from the repository root in a checkout that has oracle/_ref/libkvref.so
(built by oracle/Makefile from the reference's headers where they lie):

    python tests/golden/make_vectors.py

Every array is either an input chosen here from a fixed seed or the value the
reference's code returned for it; nothing in the file comes from the oracle or
from the library under test.  Sources of the expected values:
  layout_*      kv::Layout                      runtime/ops/PagedKv.hpp:125-232
  offset_*      richengine_kv_offset / elements runtime/metal/abi/KvExtent.h:45-111
  bf16_*, fp8_* codecs                          runtime/ops/PagedKv.hpp (floatToBFloat16, floatToFp8E4m3, ...)
  stage_*       kv::queryStage                  runtime/ops/PagedKv.hpp
  splits_*      kv::verifyAttentionSplits       runtime/ops/PagedAttention.hpp:54-95
  tiles_*       kv::prefillAttentionTiles
  chunk_*       kv::chunkedPrefillValidationError / RequiredPages
  q8_*, f8_*    whole-page quantizers           dev/tests/engine/Q8PageFormatReference.hpp:141-180,
                                                dev/tests/engine/Fp8PageFormatReference.hpp:147-186
  identity_*    engine::blockImageIdentity      runtime/engine/cache/KvCache.cpp:29-52
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import kvoracle as ko  # noqa: E402  (only ref(): the ctypes view of oracle/_ref)

H, D = 4, 256


def bf16_round(x):
    """fp32 -> nearest-even bf16 -> fp32, in numpy (inputs only)."""
    b = x.astype(np.float32).view(np.uint32)
    b = (b + 0x7FFF + ((b >> 16) & 1)) & 0xFFFF0000
    return b.astype(np.uint32).view(np.float32)


def main():
    R = ko.ref()
    if R is None:
        raise SystemExit("oracle/_ref/libkvref.so is missing: run make -C oracle ref")
    rng = np.random.default_rng(20261125)
    out = {}

    # ---- layouts: (layers, heads, dim, format) -> the 8 numbers of ref_layout
    layouts = np.array([(l, h, d, f) for f in range(4) for (l, h, d) in
                        [(16, 4, 256), (1, 1, 64), (32, 8, 128), (48, 2, 256), (2, 4, 96)]],
                       dtype=np.uint32)
    numbers = np.zeros((len(layouts), 8), dtype=np.uint64)
    for i, (l, h, d, f) in enumerate(layouts):
        R.ref_layout(int(l), int(h), int(d), int(f), numbers[i].ctypes.data_as(C.POINTER(C.c_uint64)))
    out["layout_in"], out["layout_out"] = layouts, numbers
    want_pages = np.array([1, 31, 32, 33, 500, 4096, 16383, 16384, 100000], dtype=np.uint64)
    out["layout_extent_pages_in"] = want_pages
    out["layout_extent_pages_out"] = np.array(
        [[R.ref_extent_pages_for(int(l), int(h), int(d), int(f), int(p)) for p in want_pages]
         for (l, h, d, f) in layouts], dtype=np.uint32)

    # ---- offsets: random (extent_pages, data bytes, scale bytes, layer, tensor, index)
    n = 400
    db = rng.choice([4096, 16384, 32768, 65536], n)
    sb = rng.choice([128, 512, 1024], n)
    # extents whose 16 layer regions stay below 4 GiB (offsets are 32-bit in the reference's layer POD)
    ep = (rng.random(n) * np.minimum(16383, (2 ** 32 - 1) // (32 * (db + sb)))).astype(np.int64) + 1
    layer = rng.integers(0, 16, n)
    tensor = rng.integers(0, 4, n)
    index = (rng.random(n) * ep).astype(np.int64)
    out["offset_in"] = np.stack([ep, db, sb, layer, tensor, index], 1).astype(np.uint32)
    out["offset_out"] = np.array([R.ref_kv_offset(*map(int, row)) for row in out["offset_in"]],
                                 dtype=np.uint64)
    coords = np.stack([rng.integers(0, 8, n), rng.integers(0, 32, n), rng.integers(0, 64, n),
                       rng.choice([64, 128, 256], n)], 1).astype(np.uint32)
    out["element_in"] = coords
    out["element_key"] = np.array([R.ref_key_element(*map(int, c)) for c in coords], dtype=np.uint64)
    out["element_value"] = np.array([R.ref_value_element(*map(int, c)) for c in coords], dtype=np.uint64)
    out["element_scale"] = np.array([R.ref_scale_element(int(c[0]), int(c[1])) for c in coords],
                                    dtype=np.uint64)

    # ---- codecs
    floats = np.concatenate([
        rng.standard_normal(600).astype(np.float32) * np.exp(rng.uniform(-40, 40, 600)).astype(np.float32),
        np.array([0.0, -0.0, 1.0, -1.0, 448.0, 449.0, 464.0, 480.0, 1e30, -1e30, 2.0 ** -6, 2.0 ** -7,
                  2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -10, 3e-39, np.inf, -np.inf, 65504.0, 65520.0,
                  6e-8, 5.9e-8, 3e-8], dtype=np.float32),
        (np.arange(0, 960, dtype=np.float32) / 2.0),  # every e4m3 rounding boundary up to 480
    ])
    out["codec_in"] = floats
    out["bf16_bits"] = np.array([R.ref_float_to_bf16(float(v)) for v in floats], dtype=np.uint16)
    out["fp8_codes"] = np.array([R.ref_float_to_fp8(float(v)) for v in floats], dtype=np.uint8)
    out["fp8_decode"] = np.array([R.ref_fp8_to_float(c) for c in range(256)], dtype=np.float32)
    out["stage_out"] = np.array([R.ref_query_stage(float(v)) for v in floats], dtype=np.float32)

    # ---- planning
    plan = np.array([(c, r) for c in [0, 1, 31, 32, 1000, 1023, 1024, 4096, 8191, 8192, 32767, 65536,
                                      131072, 1048576 - 16]
                     for r in [1, 2, 8, 15, 16]], dtype=np.uint32)
    out["splits_in"] = plan
    out["splits_out"] = np.array([R.ref_verify_splits(int(c), int(r)) for c, r in plan], dtype=np.uint32)
    rows = np.array([1, 7, 8, 9, 64, 2047, 2048], dtype=np.uint32)
    out["tiles_in"] = rows
    out["tiles_out"] = np.array([R.ref_prefill_tiles(int(r)) for r in rows], dtype=np.uint32)
    chunks = np.array([(0, 1, 32, 1), (0, 0, 32, 1), (0, 2049, 4096, 100), (1048576, 1, 32, 40000),
                       (1048575, 2, 32, 40000), (10, 40, 32, 2), (10, 40, 48, 2), (10, 40, 64, 1),
                       (10, 40, 64, 2), (0, 32, 4096, 1), (31, 1, 32, 1), (32, 1, 32, 1)], dtype=np.uint32)
    out["chunk_in"] = chunks
    out["chunk_error"] = np.array([R.ref_chunk_validation(*map(int, c)) for c in chunks], dtype=np.int32)
    out["chunk_pages"] = np.array([R.ref_chunk_required_pages(int(c[0]), int(c[1])) for c in chunks],
                                  dtype=np.uint32)

    # ---- whole-page quantizers: logical [token][head][d] bf16-exact fp32 rows
    page_bytes = R.ref_q8_page_bytes()
    for name, fn in (("q8", R.ref_quantize_q8_page), ("f8", R.ref_quantize_fp8_page)):
        for case, tokens in (("a", 32), ("b", 9)):
            if case == "a":  # the reference test's own inputs (q8_paged_kv_test.cc:92-110)
                t, h, d = np.meshgrid(np.arange(tokens), np.arange(H), np.arange(D), indexing="ij")
                k = 2.5 * np.sin((t * 17 + h * 31 + d).astype(np.float32) * np.float32(0.013))
                v = 1.75 * np.cos((t * 29 + h * 11 + d).astype(np.float32) * np.float32(0.017))
            else:
                k = rng.standard_normal((tokens, H, D)) * rng.choice([1e-3, 1.0, 300.0], (tokens, H, 1))
                v = rng.standard_normal((tokens, H, D))
                v[:, :, 5] *= 20
                k[0, 1, :] = 0.0
            k, v = bf16_round(k.astype(np.float32)), bf16_round(v.astype(np.float32))
            page = np.zeros(page_bytes, dtype=np.uint8)
            rc = fn(np.ascontiguousarray(k).ctypes.data_as(C.POINTER(C.c_float)),
                    np.ascontiguousarray(v).ctypes.data_as(C.POINTER(C.c_float)), tokens,
                    page.ctypes.data_as(C.POINTER(C.c_uint8)))
            assert rc == 0
            out[f"{name}_{case}_keys_bf16"] = (k.view(np.uint32) >> 16).astype(np.uint16)
            out[f"{name}_{case}_values_bf16"] = (v.view(np.uint32) >> 16).astype(np.uint16)
            out[f"{name}_{case}_page"] = page

    path = os.path.join(HERE, "reference_vectors.npz")
    # ---- image identities: span lists (sorted, disjoint) and blocks around them
    if ko.ref_image_identity(0, 32, []) is None:
        raise SystemExit("oracle/_ref/libkvref_cache.so is missing: run make -C oracle ref")
    cases, spans_flat, spans_first, answers = [], [], [0], []
    for case in range(48):
        spans, at = [], int(rng.integers(0, 70))
        for _ in range(int(rng.integers(0, 4))):
            tokens = int(rng.integers(1, 90))
            spans.append((at, tokens, int(rng.integers(1, 40)), int(rng.integers(1, 40)),
                          int(rng.integers(0, 2**63)) * 2 + int(rng.integers(0, 2)),
                          int(rng.integers(0, 2**63)) * 2 + int(rng.integers(0, 2))))
            at += tokens + int(rng.integers(0, 50))
        if case == 0:
            spans = []                                      # a text-only prompt
        if case == 1:
            spans = [(0xFFFFFFF0, 0x20, 3, 3, 5, 7)]        # a span whose 32-bit end wraps
        for begin in sorted({0, 32, 64, 96, 160, 320} | {s[0] // 32 * 32 for s in spans} |
                            {(s[0] + s[1]) // 32 * 32 for s in spans}):
            cases.append((len(spans_first) - 1, begin & 0xFFFFFFFFFFFF, 32))
            answers.append(ko.ref_image_identity(begin, 32, spans))
        cases.append((len(spans_first) - 1, 7, 100))         # a block that is not a page
        answers.append(ko.ref_image_identity(7, 100, spans))
        spans_flat += spans
        spans_first.append(len(spans_flat))
    out["identity_spans"] = np.array(spans_flat, dtype=np.uint64).reshape(-1, 6)
    out["identity_spans_first"] = np.array(spans_first, dtype=np.uint32)
    out["identity_cases"] = np.array(cases, dtype=np.uint64)      # (span list, block begin, block tokens)
    out["identity_out"] = np.array(answers, dtype=np.uint64)      # (lo, hi)

    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
