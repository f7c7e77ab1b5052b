"""ctypes face of the CPU oracle -- TEST INFRASTRUCTURE ONLY.

Only tests, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU-baseline leg may
import this module.  The product (``richengine_amd``) never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

INT8, BF16, INT4, FP8 = 1, 2, 3, 4
KEYS, KEY_SCALES, VALUES, VALUE_SCALES = 0, 1, 2, 3
PAGE = 32
FORMAT_NAMES = {INT8: "int8", BF16: "bf16", INT4: "int4", FP8: "fp8e4m3"}
BYTES_PER_TOKEN_LAYER = {INT4: 1056, INT8: 2080, FP8: 2080, BF16: 4096}


class Layout(C.Structure):
    _fields_ = [("layers", C.c_uint32), ("kv_heads", C.c_uint32), ("head_dim", C.c_uint32),
                ("format", C.c_uint32), ("score_scale", C.c_float)]


class KvLayer(C.Structure):
    _fields_ = [("extent_pages", C.c_uint32), ("offset", C.c_uint32)]


class ChunkParams(C.Structure):
    _fields_ = [("committed_tokens", C.c_uint32), ("chunk_tokens", C.c_uint32),
                ("chunk_stride", C.c_uint32), ("page_table_entries", C.c_uint32),
                ("kv", KvLayer)]


class PrefillParams(C.Structure):
    _fields_ = [("committed_tokens", C.c_uint32), ("rows", C.c_uint32),
                ("chunk_stride", C.c_uint32), ("page_table_entries", C.c_uint32),
                ("kv", KvLayer), ("split_count", C.c_uint32), ("score_scale", C.c_float)]


class VerifyParams(C.Structure):
    _fields_ = [("committed_tokens", C.c_uint32), ("page_table_entries", C.c_uint32),
                ("kv", KvLayer), ("split_count", C.c_uint32), ("slot_splits", C.c_uint32),
                ("active_rows", C.c_uint32), ("row_capacity", C.c_uint32),
                ("score_scale", C.c_float)]


class PageCopy(C.Structure):
    _fields_ = [("from_", C.c_uint32), ("to", C.c_uint32)]


class PoolSnapshot(C.Structure):
    _fields_ = [("pages_allocated", C.c_uint32), ("pages_free", C.c_uint32),
                ("pages_active", C.c_uint32), ("pages_prefix", C.c_uint32),
                ("allocated_bytes", C.c_uint64), ("reclaimable_bytes", C.c_uint64),
                ("extent_allocations", C.c_uint64), ("extent_releases", C.c_uint64),
                ("extent_compactions", C.c_uint64), ("pages_moved", C.c_uint64)]


def build(force=False):
    """Compiles the oracle (and oracle/_ref when the reference checkout exists)."""
    so = os.path.join(_HERE, "libkvoracle.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", _HERE, "-s", "libkvoracle.so"] + (["-B"] if force else []))
    return so


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        _declare(_lib)
    return _lib


def set_threads(threads):
    """Threads the oracle's attention functions may use (1 = the scalar baseline)."""
    lib().ko_set_threads(int(threads))


_ref_cache = None


def ref_image_identity(block_begin, block_tokens, spans):
    """(lo, hi) from the reference's own blockImageIdentity (oracle/_ref/libkvref_cache.so:
    runtime/engine/cache/KvCache.cpp compiled where it lies), or None where it was not built.
    spans: (offset, tokens, grid height, grid width, digest lo, digest hi) tuples."""
    global _ref_cache
    if _ref_cache is None:
        path = os.path.join(_HERE, "_ref", "libkvref_cache.so")
        if not os.path.exists(path):
            return None
        _ref_cache = C.CDLL(path)
        _ref_cache.ref_image_identity.argtypes = [C.c_uint64, C.c_uint32, C.c_void_p, C.c_uint32,
                                                  C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
        _ref_cache.ref_image_identity.restype = None
    words = np.array([w for span in spans for w in span], dtype=np.uint64)
    lo, hi = C.c_uint64(), C.c_uint64()
    _ref_cache.ref_image_identity(block_begin, block_tokens, words.ctypes.data_as(C.c_void_p),
                                  len(spans), C.byref(lo), C.byref(hi))
    return lo.value, hi.value


def ref():
    """The reference's own host code (oracle/_ref), or None where it was not built."""
    global _ref
    if _ref is None:
        path = os.path.join(_HERE, "_ref", "libkvref.so")
        if not os.path.exists(path):
            return None
        r = C.CDLL(path)
        u32, u64, f32 = C.c_uint32, C.c_uint64, C.c_float
        r.ref_layout.argtypes = [u32, u32, u32, u32, C.POINTER(u64)]
        r.ref_extent_pages_for.argtypes = [u32, u32, u32, u32, u64]
        r.ref_extent_pages_for.restype = u32
        for name in ("ref_key_element", "ref_value_element"):
            getattr(r, name).argtypes = [u32] * 4
            getattr(r, name).restype = u64
        r.ref_scale_element.argtypes = [u32, u32]
        r.ref_scale_element.restype = u64
        r.ref_kv_offset.argtypes = [u32] * 6
        r.ref_kv_offset.restype = u64
        r.ref_kv_layer.argtypes = [u32] * 4
        r.ref_kv_layer.restype = u64
        r.ref_page_entry.argtypes = [u64, u32]
        r.ref_page_entry.restype = u64
        r.ref_float_to_bf16.argtypes = [f32]
        r.ref_float_to_bf16.restype = C.c_uint16
        r.ref_bf16_to_float.argtypes = [C.c_uint16]
        r.ref_bf16_to_float.restype = f32
        r.ref_float_to_fp8.argtypes = [f32]
        r.ref_float_to_fp8.restype = C.c_uint8
        r.ref_fp8_to_float.argtypes = [C.c_uint8]
        r.ref_fp8_to_float.restype = f32
        r.ref_query_stage.argtypes = [f32]
        r.ref_query_stage.restype = f32
        r.ref_verify_splits.argtypes = [u32, u32]
        r.ref_verify_splits.restype = u32
        r.ref_prefill_tiles.argtypes = [u32]
        r.ref_prefill_tiles.restype = u32
        r.ref_chunk_validation.argtypes = [u32] * 4
        r.ref_chunk_validation.restype = C.c_int
        r.ref_chunk_required_pages.argtypes = [u32, u32]
        r.ref_chunk_required_pages.restype = u32
        r.ref_param_sizes.argtypes = [u32]
        r.ref_param_sizes.restype = u32
        for name in ("ref_quantize_q8_page", "ref_quantize_fp8_page"):
            getattr(r, name).argtypes = [C.c_void_p, C.c_void_p, u32, C.c_void_p]
            getattr(r, name).restype = C.c_int
        r.ref_q8_page_bytes.restype = u64
        _ref = r
    return _ref


def _declare(L):
    u32, u64, f32, vp = C.c_uint32, C.c_uint64, C.c_float, C.c_void_p
    LP = C.POINTER(Layout)
    for name in ("ko_elements_per_layer_page", "ko_data_bytes_per_layer_page",
                 "ko_scale_bytes_per_layer_page", "ko_bytes_per_layer_page",
                 "ko_bytes_per_model_page"):
        getattr(L, name).argtypes = [LP]
        getattr(L, name).restype = u64
    for name in ("ko_extent_alignment_pages", "ko_minimum_extent_pages",
                 "ko_maximum_extent_pages"):
        getattr(L, name).argtypes = [LP]
        getattr(L, name).restype = u32
    L.ko_layout_valid.argtypes = [LP]
    L.ko_extent_pages_for.argtypes = [LP, u64]
    L.ko_extent_pages_for.restype = u32
    for name in ("ko_key_element", "ko_value_element"):
        getattr(L, name).argtypes = [u32] * 4
        getattr(L, name).restype = u64
    L.ko_scale_element.argtypes = [u32, u32]
    L.ko_scale_element.restype = u64
    L.ko_kv_offset.argtypes = [u32] * 6
    L.ko_kv_offset.restype = u64
    L.ko_kv_layer_of.argtypes = [u32] * 4
    L.ko_kv_layer_of.restype = KvLayer
    L.ko_page_entry.argtypes = [u64, u32]
    L.ko_page_entry.restype = u64
    L.ko_float_to_bf16.argtypes = [f32]
    L.ko_float_to_bf16.restype = C.c_uint16
    L.ko_bf16_to_float.argtypes = [C.c_uint16]
    L.ko_bf16_to_float.restype = f32
    L.ko_float_to_fp8e4m3.argtypes = [f32]
    L.ko_float_to_fp8e4m3.restype = C.c_uint8
    L.ko_fp8e4m3_to_float.argtypes = [C.c_uint8]
    L.ko_fp8e4m3_to_float.restype = f32
    L.ko_round_to_f16.argtypes = [f32]
    L.ko_round_to_f16.restype = f32
    L.ko_verify_splits.argtypes = [u32, u32]
    L.ko_verify_splits.restype = u32
    L.ko_prefill_tiles.argtypes = [u32]
    L.ko_prefill_tiles.restype = u32
    L.ko_prefill_splits.argtypes = [u32]
    L.ko_prefill_splits.restype = u32
    L.ko_chunk_validation.argtypes = [C.POINTER(ChunkParams)]
    L.ko_chunk_required_pages.argtypes = [C.POINTER(ChunkParams)]
    L.ko_chunk_required_pages.restype = u32
    L.ko_prefill_workspace.argtypes = [u32, u32, u32, u32, C.POINTER(u64), C.POINTER(u64)]
    L.ko_prefill_workspace_bound.argtypes = [u32, u32, u32, C.POINTER(u64), C.POINTER(u64)]
    L.ko_verify_workspace.argtypes = [u32, u32, u32, u32, C.POINTER(u64), C.POINTER(u64)]
    L.ko_store_create.argtypes = [LP, u32, u32]
    L.ko_store_create.restype = vp
    L.ko_store_create_host.argtypes = [LP, u32, u32]
    L.ko_store_create_host.restype = vp
    L.ko_store_destroy.argtypes = [vp]
    L.ko_store_allocate_extent.argtypes = [vp, u32]
    L.ko_store_release_extent.argtypes = [vp, u32]
    L.ko_store_extent.argtypes = [vp, u32]
    L.ko_store_extent.restype = vp
    L.ko_store_extent_bytes.argtypes = [vp]
    L.ko_store_extent_bytes.restype = u64
    L.ko_store_extent_pages.argtypes = [vp]
    L.ko_store_extent_pages.restype = u32
    L.ko_store_layer.argtypes = [vp, u32]
    L.ko_store_layer.restype = KvLayer
    L.ko_store_write_entries.argtypes = [vp, vp, u32, u32, vp]
    L.ko_store_copy_pages.argtypes = [vp, vp, u32]
    L.ko_store_page_read.argtypes = [vp, u32, vp]
    L.ko_store_page_write.argtypes = [vp, u32, vp]
    L.ko_store_chunk.argtypes = [u32, u32, u32, vp, vp, vp, C.POINTER(ChunkParams)]
    L.ko_store_verify.argtypes = [u32, u32, u32, vp, vp, vp, vp, u32, u32]
    L.ko_attention_tile.argtypes = [u32, u32, u32, u32, u32, vp, vp, KvLayer, u32, u32, u32, u32,
                                    u32, vp, vp, u64, vp, f32]
    L.ko_attention_reduce_row.argtypes = [u32, u32, u32, vp, vp, u32, u32, u32, u64, u32, vp, vp]
    L.ko_attention_reduce_row.restype = None
    L.ko_attention_flips.argtypes = [C.c_int64, vp, u32, C.c_float, C.c_int]
    L.ko_attention_flips.restype = None
    L.ko_attention_flips_applied.argtypes = []
    L.ko_attention_flips_applied.restype = u32
    L.ko_attention_row_weights.argtypes = [u32, u32, u32, vp, vp, KvLayer, u32, u32, u32, u32, vp,
                                           C.c_float, vp]
    L.ko_attention_row_weights.restype = None
    L.ko_attend_prefill.argtypes = [u32, u32, u32, u32, vp, vp, vp, vp, C.POINTER(PrefillParams)]
    L.ko_attend_verify.argtypes = [u32, u32, u32, u32, vp, vp, vp, vp, vp, u32, vp]
    L.ko_compact_tree.argtypes = [u32, u32, u32, vp, vp, vp, vp, u32, u32]
    L.ko_qkv_prepare.argtypes = [u32, u32, u32, u32, C.c_int, C.c_int, C.c_float, u32, u32, vp, vp, vp,
                                 vp, vp, vp, vp, vp]
    L.ko_qkv_prepare.restype = None
    L.ko_sigmoid.argtypes = [C.c_float]
    L.ko_sigmoid.restype = C.c_float
    L.ko_attention_hidden.argtypes = [u32, u32, u32, u32, u32, u32, vp, vp, vp]
    L.ko_attention_hidden.restype = None
    L.ko_pool_create.argtypes = [u32, u64, u32, u32, u32]
    L.ko_pool_create.restype = vp
    L.ko_pool_destroy.argtypes = [vp]
    L.ko_pool_set_growth_blocked.argtypes = [vp, C.c_int]
    L.ko_pool_set_refused_extent.argtypes = [vp, C.c_int64]
    L.ko_pool_set_budget_pages.argtypes = [vp, u32]
    L.ko_pool_acquire.argtypes = [vp, u32, vp]
    L.ko_pool_retain.argtypes = [vp, u32, C.c_int]
    L.ko_pool_release.argtypes = [vp, u32, C.c_int]
    L.ko_pool_page_active.argtypes = [vp, u32]
    L.ko_pool_reclaim_empty.argtypes = [vp, C.c_int, u32]
    L.ko_pool_reclaim_empty.restype = u64
    L.ko_pool_compact_extent.argtypes = [vp, vp, u32, C.POINTER(u32), vp, vp, C.POINTER(u32)]
    L.ko_pool_snapshot_get.argtypes = [vp, C.POINTER(PoolSnapshot)]
    L.ko_pool_content.argtypes = [vp, u32]
    L.ko_pool_content.restype = u64
    L.ko_pool_set_content.argtypes = [vp, u32, u64]
    L.ko_pool_extent_allocated.argtypes = [vp, u32]


def ptr(a):
    """Address of a numpy array's data (None passes NULL)."""
    return None if a is None else a.ctypes.data


# ----------------------------------------------------------------- bf16 ---
def f32_to_bf16(x):
    """Round-to-nearest-even fp32 -> bf16 bits (numpy, vectorised; NaN kept)."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    special = (b & 0x7F800000) == 0x7F800000
    upper = (b >> 16).astype(np.uint16)
    fix = special & ((b & 0x007FFFFF) != 0) & ((upper & 0x7F) == 0)
    rounded = ((b.astype(np.uint64) + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)
    return np.where(special, np.where(fix, upper | 1, upper), rounded).astype(np.uint16)


def bf16_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# ---------------------------------------------------------------- store ---
class Store:
    """Host page storage laid out exactly like the device pool's extents."""

    def __init__(self, layers, kv_heads, head_dim, fmt, page_count, extent_pages,
                 score_scale=0.0, aligned=False):
        self.layout = Layout(layers, kv_heads, head_dim, fmt, score_scale)
        create = lib().ko_store_create if aligned else lib().ko_store_create_host
        self.h = create(C.byref(self.layout), page_count, extent_pages)
        if not self.h:
            raise ValueError("invalid KV store geometry")
        self.page_count, self.extent_pages = page_count, extent_pages
        self.extent_bytes = lib().ko_store_extent_bytes(self.h)
        self.bytes_per_page = lib().ko_bytes_per_model_page(C.byref(self.layout))

    def close(self):
        if self.h:
            lib().ko_store_destroy(self.h)
            self.h = None

    def __del__(self):
        self.close()

    def allocate(self, extent):
        return lib().ko_store_allocate_extent(self.h, extent)

    def release(self, extent):
        return lib().ko_store_release_extent(self.h, extent)

    def extent(self, extent):
        """The extent's bytes as a numpy view (no copy)."""
        p = lib().ko_store_extent(self.h, extent)
        if not p:
            return None
        buf = (C.c_uint8 * self.extent_bytes).from_address(p)
        return np.frombuffer(buf, dtype=np.uint8)

    def layer(self, layer):
        return lib().ko_store_layer(self.h, layer)

    def entries(self, pages, first=0):
        pages = np.ascontiguousarray(pages, dtype=np.uint32)
        table = np.zeros(len(pages), dtype=np.uint64)
        rc = lib().ko_store_write_entries(self.h, ptr(pages), len(pages), first, ptr(table))
        if rc:
            raise RuntimeError(f"write_entries failed: {rc}")
        return table

    def copy_pages(self, copies):
        arr = (PageCopy * len(copies))(*[PageCopy(a, b) for a, b in copies])
        return lib().ko_store_copy_pages(self.h, arr, len(copies))

    def page_read(self, page):
        out = np.empty(self.bytes_per_page, dtype=np.uint8)
        rc = lib().ko_store_page_read(self.h, page, ptr(out))
        if rc:
            raise RuntimeError(f"page_read failed: {rc}")
        return out

    def page_write(self, page, data):
        data = np.ascontiguousarray(data, dtype=np.uint8)
        assert data.size == self.bytes_per_page
        return lib().ko_store_page_write(self.h, page, ptr(data))


def store_chunk(fmt, kv_heads, head_dim, chunk_keys, chunk_values, table, params):
    return lib().ko_store_chunk(fmt, kv_heads, head_dim, ptr(chunk_keys), ptr(chunk_values),
                                ptr(table), C.byref(params))


def _table_ptrs(tables):
    arr = (C.c_void_p * len(tables))(*[t.ctypes.data for t in tables])
    return arr


def store_verify(fmt, kv_heads, head_dim, chunk_keys, chunk_values, tables, params, max_rows=15):
    arr = (ChunkParams * len(params))(*params)
    return lib().ko_store_verify(fmt, kv_heads, head_dim, ptr(chunk_keys), ptr(chunk_values),
                                 _table_ptrs(tables), arr, len(params), max_rows)


def attend_prefill(fmt, kv_heads, group, head_dim, queries, table, params, want_f32=True):
    out = np.zeros(queries.shape, dtype=np.uint16)
    f32 = np.zeros(queries.shape, dtype=np.float32) if want_f32 else None
    ok = lib().ko_attend_prefill(fmt, kv_heads, group, head_dim, ptr(queries), ptr(out), ptr(f32),
                                 ptr(table), C.byref(params))
    return ok, out, f32


def attend_verify(fmt, kv_heads, group, head_dim, queries, tables, params, row_masks=None,
                  want_f32=True):
    out = np.zeros(queries.shape, dtype=np.uint16)
    f32 = np.zeros(queries.shape, dtype=np.float32) if want_f32 else None
    arr = (VerifyParams * len(params))(*params)
    n = lib().ko_attend_verify(fmt, kv_heads, group, head_dim, ptr(queries), ptr(out), ptr(f32),
                               _table_ptrs(tables), arr, len(params), ptr(row_masks))
    return n, out, f32


def qkv_prepare(kv_heads, group, head_dim, rotary_pairs, query_gate, eps, tokens, stride, packed,
                q_norm, k_norm, rope_cos, rope_sin):
    """One lane: (queries [kv head][stride][g][D], chunk_keys [kv head][stride][D],
    chunk_values [kv head][D][stride]) as bf16 bit patterns.  Norm weights: None, uint16 (bf16
    bits) or float32 arrays."""
    queries = np.zeros((kv_heads, stride, group, head_dim), dtype=np.uint16)
    keys = np.zeros((kv_heads, stride, head_dim), dtype=np.uint16)
    values = np.zeros((kv_heads, head_dim, stride), dtype=np.uint16)
    norm_f32 = int(q_norm is not None and q_norm.dtype == np.float32)
    lib().ko_qkv_prepare(kv_heads, group, head_dim, rotary_pairs, int(query_gate), norm_f32, eps,
                         tokens, stride, ptr(packed), ptr(q_norm), ptr(k_norm), ptr(rope_cos),
                         ptr(rope_sin), ptr(queries), ptr(keys), ptr(values))
    return queries, keys, values


def attention_hidden(kv_heads, group, head_dim, rows, attention, packed_qkv=None):
    """hidden [lane][rows][query head][D] from staged rows [lane][kv head][stride][g][D]."""
    lanes, _, row_stride = attention.shape[:3]
    hidden = np.zeros((lanes, rows, kv_heads * group, head_dim), dtype=np.uint16)
    lib().ko_attention_hidden(kv_heads, group, head_dim, lanes, rows, row_stride, ptr(attention),
                              ptr(packed_qkv), ptr(hidden))
    return hidden


def compact_tree(fmt, kv_heads, head_dim, tables, params, retained_path, retained_count,
                 path_stride):
    arr = (ChunkParams * len(params))(*params)
    return lib().ko_compact_tree(fmt, kv_heads, head_dim, _table_ptrs(tables), arr,
                                 ptr(retained_path), ptr(retained_count), len(params), path_stride)


# ------------------------------------------------ one tile, and "what if" rows ---
def attention_tile_rows(fmt, kv_heads, group, head_dim, tile_queries, table, kv, head, committed,
                        active, splits, capacity, masks=None, score_scale=0.0, only_row=None):
    """The oracle's attention of one tile (capacity rows x group fused rows) of one KV head: every
    split's partial tile, then the fixed-order merge of each live fused row.  tile_queries: bf16
    [capacity * group, D].  Returns (bf16, fp32) outputs of that shape; rows past `active` are
    zeros.  only_row: merge that fused row alone (the others stay zero)."""
    L = lib()
    M, D = capacity * group, head_dim
    tile_queries = np.ascontiguousarray(tile_queries, dtype=np.uint16).reshape(M, D)
    partials = np.zeros((splits, M, D), dtype=np.float32)
    statistics = np.zeros((splits, M, 2), dtype=np.float32)
    mask_ptr = ptr(np.ascontiguousarray(masks, dtype=np.uint32)) if masks is not None else None
    for split in range(splits):
        L.ko_attention_tile(fmt, kv_heads, group, D, capacity, ptr(tile_queries), ptr(table), kv,
                            head, committed, active, splits, split, ptr(partials),
                            ptr(statistics), split, mask_ptr, score_scale)
    out = np.zeros((M, D), dtype=np.uint16)
    out32 = np.zeros((M, D), dtype=np.float32)
    for row in (range(M) if only_row is None else [only_row]):
        L.ko_attention_reduce_row(group, D, capacity, ptr(partials), ptr(statistics), committed,
                                  active, splits, 0, row, ptr(out[row]), ptr(out32[row]))
    return out, out32


# How far (relative) the unrounded weight of a token may lie from a rounding boundary for the
# other rounding to count as explained.  It stands for the deviation between a score of the
# matrix-core kernels and the oracle's (another order of the sums of q.k in fp32): a score that
# is off by d moves its probability by d, relatively.  That deviation is measured, not argued:
# every split reports the maximum of its scores and the sum of its probabilities, on both sides,
# and tests/test_gpu_score_deviation.py compares them over 8000 split statistics per format --
# long histories with 20x outlier channels in the keys, one-row decode, 8-row chains and lanes of
# 12 and 16 rows (the kernels of wide lanes), plain
# queries and queries that carry the keys' outlier channels too (scores of a hundred and more,
# harsher than anything else the suite holds).  Worst |max - max| it found:
#              plain queries   outlier queries
#   int4         4.8e-05          1.8e-04
#   int8         1.9e-06          1.2e-04
#   bf16         1.1e-05          3.4e-04
#   fp8          5.7e-06          2.8e-04
# The slack of a format is twice its worst figure; the test holds every new measurement to half
# of the slack and prints what it measured in the run's summary.  A bf16 place is 3.9e-3 to
# 7.8e-3 relative, so one weight in ten lies this close to a boundary; an fp16 place (the
# weights on fp8 pages) is 4.9e-4 to 9.8e-4, so on those pages nearly every weight does, which
# is what the measurement says: at such scores the fp16 rounding of a weight is not determined
# by the inputs alone.
FLIP_SLACK = {INT4: 3.7e-4, INT8: 2.5e-4, BF16: 6.8e-4, FP8: 5.5e-4}


def flip_slack(fmt):
    """The measured score deviation of the format's matrix-core kernels, doubled (FLIP_SLACK)."""
    return FLIP_SLACK[fmt]


def rounding_flip_rows(fmt, kv_heads, group, head_dim, tile_queries, table, kv, head, committed,
                       active, splits, capacity, fused_row, masks=None, score_scale=0.0, top=64,
                       slack=None, together=2):
    """What one fused row of a tile would be had the rounding of some of its heaviest
    probabilities fallen the other way.  Of the row's `top` heaviest tokens (softmax weight x
    value scale) only those count whose unrounded weight lies within `slack` (relative) of a
    rounding boundary of its format (bf16; fp16 on fp8 pages): for every set of at most
    `together` of them the oracle recomputes the row with those weights on the other side of
    their boundaries.  Yields (tokens, len(tokens), bf16 row bits).

    How much one turned rounding moves a row: a place of a weight in [0.25, 0.5) is 2^-9, and
    the row is a sum of value rows with weights w, so it moves by about 2^-9 / sqrt(sum w^2) --
    1e-3 to 3e-3 when the attention is spread over some ten heavy tokens, each of which can be
    the one.  Hence `top` reaches well past the few heaviest: a row over 150 tokens was moved
    past the tolerance by its 40th heaviest token (weight 8.4e-3, 1.1e-7 from a tie), exactly one
    place of that weight in one split's partial row and nothing else.

    A kernel that sums q.k in another order than this oracle differs from it in the last bits of
    a score, and so in the rounding of a probability that sits on a rounding boundary; a token
    that carries much of the row then moves the whole row by up to half a place.  A row that is
    farther from the oracle than the tolerance, but within it of one of these rows, is explained
    by exactly that; any other difference is not."""
    import itertools
    L = lib()
    if slack is None:
        slack = flip_slack(fmt)
    M, D = capacity * group, head_dim
    tile_queries = np.ascontiguousarray(tile_queries, dtype=np.uint16).reshape(M, D)
    row = fused_row // group
    weights = np.zeros(committed + active, dtype=np.float32)
    mask_ptr = ptr(np.ascontiguousarray(masks, dtype=np.uint32)) if masks is not None else None
    L.ko_attention_row_weights(fmt, kv_heads, D, ptr(tile_queries[fused_row]), ptr(table), kv, head,
                               committed, active, row, mask_ptr, score_scale, ptr(weights))
    heaviest = [int(t) for t in np.argsort(-weights, kind="stable")[:top] if weights[t] > 0]

    def recompute(tokens):
        arr = np.array(tokens, dtype=np.uint32)
        L.ko_attention_flips(fused_row, ptr(arr), len(arr), slack, 1)
        try:
            bits, _ = attention_tile_rows(fmt, kv_heads, group, D, tile_queries, table, kv, head,
                                          committed, active, splits, capacity, masks, score_scale,
                                          only_row=fused_row)
            return bits[fused_row], L.ko_attention_flips_applied()
        finally:
            L.ko_attention_flips(-1, None, 0, 0.0, 0)

    near = []                                 # which of them sit on a boundary at all
    for first in range(0, len(heaviest), 32):  # the tile takes 32 tokens to turn at a time
        some = heaviest[first:first + 32]
        _, applied = recompute(some)
        near += [t for i, t in enumerate(some) if applied >> i & 1]
    for size in range(1, min(together, len(near)) + 1):
        for tokens in itertools.combinations(near, size):
            bits, _ = recompute(list(tokens))
            yield tokens, size, bits
