"""Helpers shared by the tests: reference-held input patterns and pool fixtures."""
import ctypes as C

import numpy as np

from oracle import kvoracle as ko


# -- closed-form patterns the reference's own tests use -----------------------
def key_pattern(token, head, d, variant=0):
    """dev/tests/engine/q8_chunked_prefill_metal_test.mm:92-100"""
    c = ((token + 13 * variant) * 37 + head * 101 + d * 17 + (token + variant) * d * 3) % 2003 - 1001
    return np.float32(c) / np.float32(2002.0)


def value_pattern(token, head, d, variant=0):
    """dev/tests/engine/q8_chunked_prefill_metal_test.mm:102-110"""
    c = ((token + 17 * variant) * 53 + head * 79 + d * 29 + (token + variant) * d * 5) % 2011 - 1005
    return np.float32(c) / np.float32(1005.0)


def query_pattern(row, head, d):
    """dev/tests/engine/q8_chunked_prefill_metal_test.mm:112-119"""
    c = (row * 43 + head * 67 + d * 11 + head * d * 7) % 1019 - 509
    return np.float32(c) / np.float32(2036.0)


def plan_key_code(token, head, d, lane, int4):
    """dev/tests/engine/paged_attention_plan_test.mm:358-364"""
    m = 15 if int4 else 255
    return (token * 37 + head * 101 + d * 17 + token * d * 3 + lane * 7) % m - (7 if int4 else 127)


def plan_value_code(token, head, d, lane, int4):
    """dev/tests/engine/paged_attention_plan_test.mm:365-371"""
    m = 15 if int4 else 255
    return (token * 53 + head * 79 + d * 29 + token * d * 5 + lane * 19) % m - (7 if int4 else 127)


def plan_query(row, head, d):
    """dev/tests/engine/paged_attention_plan_test.mm:421-425"""
    return np.float32((row * 43 + head * 67 + d * 11 + head * d * 7) % 1019 - 509) / np.float32(1018.0)


# -- pool fixtures -------------------------------------------------------------
def spread(pages):
    """Three or more extents of a page count that is not a power of two, as
    dev/tuning/HostKvExtents.hpp:53-57, so a table crosses extents."""
    ep = min(max((pages + 2) // 3, 3), ko.PAGE * 512 - 1)
    if ep & (ep - 1) == 0:
        ep += 1
    return ep, max(3, (pages + ep - 1) // ep)


def mixed_pages(extent_pages, extents, count, seed):
    """First and last page of every extent first, then the others, each group
    shuffled (dev/tuning/HostKvExtents.hpp:135-151; our own seeded shuffle)."""
    rng = np.random.default_rng(seed)
    pages = np.arange(extent_pages * extents)
    idx = pages % extent_pages
    boundary = pages[(idx == 0) | (idx == extent_pages - 1)]
    interior = pages[(idx != 0) & (idx != extent_pages - 1)]
    rng.shuffle(boundary)
    rng.shuffle(interior)
    out = np.concatenate([boundary, interior])[:count]
    assert len(out) == count
    return out.astype(np.uint32)


def make_store(fmt, kv_heads, head_dim, layers, pages_needed, one_extent=False):
    ep, n = spread(pages_needed + 2)
    if one_extent:
        ep, n = ep * n, 1
    s = ko.Store(layers, kv_heads, head_dim, fmt, ep * n, ep)
    for e in range(n):
        assert s.allocate(e) == 0
    return s


def slab_views(store, layer, page):
    """numpy views of one page's four tensors in one layer of an oracle store."""
    L = ko.lib()
    lay = store.layout
    db = L.ko_data_bytes_per_layer_page(C.byref(lay))
    sb = L.ko_scale_bytes_per_layer_page(C.byref(lay))
    ext = store.extent(page // store.extent_pages)
    idx = page % store.extent_pages
    out = []
    for tensor in range(4):
        size = sb if tensor % 2 else db
        off = L.ko_kv_offset(store.extent_pages, db, sb, layer, tensor, idx)
        out.append(ext[off:off + size])
    return out


def unpack_int4(data, kv_heads, head_dim):
    """[head][token][d] signed codes from a page's packed bytes (independent of
    the oracle's own nibble reader)."""
    b = data.reshape(kv_heads, 32, head_dim // 2)
    lo = (b & 0xF).astype(np.int8)
    hi = (b >> 4).astype(np.int8)
    lo = np.where(lo > 7, lo - 16, lo)
    hi = np.where(hi > 7, hi - 16, hi)
    return np.stack([lo, hi], axis=-1).reshape(kv_heads, 32, head_dim)


def page_codes(store, layer, page):
    """(K codes [H][32][D] float, K scales [H][32], V codes [H][32][D], V scales)
    decoded with numpy only."""
    lay = store.layout
    H, D, fmt = lay.kv_heads, lay.head_dim, lay.format
    k, ks, v, vs = slab_views(store, layer, page)
    if fmt == ko.INT4:
        kc, vc = unpack_int4(k, H, D), unpack_int4(v, H, D)
    elif fmt == ko.INT8:
        kc = k.view(np.int8).reshape(H, 32, D)
        vc = v.view(np.int8).reshape(H, D, 32).transpose(0, 2, 1)
    elif fmt == ko.FP8:
        lut = np.array([ko.lib().ko_fp8e4m3_to_float(c) for c in range(256)], dtype=np.float32)
        kc = lut[k.reshape(H, 32, D)]
        vc = lut[v.reshape(H, D, 32).transpose(0, 2, 1)]
    else:
        kc = ko.bf16_to_f32(k.view(np.uint16)).reshape(H, 32, D)
        vc = ko.bf16_to_f32(v.view(np.uint16)).reshape(H, D, 32).transpose(0, 2, 1)
    if fmt == ko.BF16:
        ones = np.ones((H, 32), dtype=np.float32)
        return kc.astype(np.float32), ones, vc.astype(np.float32), ones
    return (kc.astype(np.float32), ks.view(np.float32).reshape(H, 32).copy(),
            vc.astype(np.float32), vs.view(np.float32).reshape(H, 32).copy())


def chunk_buffers(keys_f32, values_f32, stride):
    """bf16 chunk staging from logical [head][token][d] fp32 rows:
    keys [head][stride][D] (token-major), values [head][D][stride]
    (dimension-major) -- common/paged_store_row.h:31-41."""
    H, T, D = keys_f32.shape
    ck = np.zeros((H, stride, D), dtype=np.uint16)
    cv = np.zeros((H, D, stride), dtype=np.uint16)
    ck[:, :T, :] = ko.f32_to_bf16(keys_f32).reshape(H, T, D)
    cv[:, :, :T] = ko.f32_to_bf16(values_f32).reshape(H, T, D).transpose(0, 2, 1)
    return ck, cv


def dense_attention_f64(q, kc, ks, vc, vs, limits, score_scale):
    """fp64 softmax(q k^T) v over dequantised history.
    q [R][D]; kc/vc [T][D] codes; ks/vs [T]; limits [R] = visible tokens per row
    (or a boolean [R][T] admission matrix)."""
    k = kc.astype(np.float64) * ks.astype(np.float64)[:, None]
    v = vc.astype(np.float64) * vs.astype(np.float64)[:, None]
    s = (q.astype(np.float64) @ k.T) * float(score_scale)
    T = k.shape[0]
    limits = np.asarray(limits)
    admit = limits if limits.ndim == 2 else np.arange(T)[None, :] < limits[:, None]
    s = np.where(admit, s, -np.inf)
    s = s - s.max(axis=1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=1, keepdims=True)
    return p @ v


def rel_l2(a, b):
    """Per-row ||a-b||2 / ||b||2 (rows on the last axis)."""
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    den = np.linalg.norm(b, axis=-1)
    num = np.linalg.norm(a - b, axis=-1)
    return np.where(den > 0, num / np.where(den > 0, den, 1), num)
