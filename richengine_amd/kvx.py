"""ctypes binding of include/kvx.h.

There is no CPU fallback: every hot-path call goes to the HIP library, and
loading fails loudly when ``libkvx.so`` is missing.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# KVX_LIB_PATH selects another build of the same library (profiling variants).
LIB_PATH = os.environ.get("KVX_LIB_PATH") or os.path.join(HERE, "libkvx.so")

INT8, BF16, INT4, FP8 = 1, 2, 3, 4
KEYS, KEY_SCALES, VALUES, VALUE_SCALES = 0, 1, 2, 3
OK, EINVAL, ESTATE, ENOMEM, ERANGE, EDEVICE = 0, -1, -2, -3, -4, -5
PAGE = 32
ALL_LAYERS = 0xFFFFFFFF
BYTES_PER_TOKEN_LAYER = {INT4: 1056, INT8: 2080, FP8: 2080, BF16: 4096}

SYMBOLS = [
    "kvx_last_error", "kvx_layout_valid", "kvx_layout_data_bytes_per_layer_page",
    "kvx_layout_scale_bytes_per_layer_page", "kvx_layout_bytes_per_layer_page",
    "kvx_layout_bytes_per_model_page", "kvx_layout_extent_alignment_pages",
    "kvx_layout_minimum_extent_pages", "kvx_layout_maximum_extent_pages",
    "kvx_layout_extent_pages_for", "kvx_layout_largest_extent_pages", "kvx_kv_offset",
    "kvx_verify_splits", "kvx_prefill_splits", "kvx_prefill_plan", "kvx_prefill_plan_batch", "kvx_decode_splits", "kvx_chunk_validation",
    "kvx_prefill_workspace", "kvx_prefill_workspace_for", "kvx_prefill_workspace_bound", "kvx_verify_workspace",
    "kvx_attend_workspace_bytes", "kvx_storage_create", "kvx_storage_destroy",
    "kvx_storage_page_count", "kvx_storage_extent_pages", "kvx_storage_bytes_per_page",
    "kvx_storage_extent_bytes", "kvx_storage_allocated_bytes", "kvx_storage_is_allocated",
    "kvx_storage_allocate_extent", "kvx_storage_release_extent", "kvx_storage_set_budget",
    "kvx_storage_layer", "kvx_storage_entries", "kvx_storage_write_entries",
    "kvx_storage_page_read", "kvx_storage_page_write", "kvx_storage_extent_read",
    "kvx_storage_extent_write", "kv_page_copy", "kvx_pool_create", "kvx_pool_destroy",
    "kvx_pool_acquire", "kvx_pool_retain", "kvx_pool_release", "kvx_pool_page_active",
    "kvx_pool_free_pages", "kvx_pool_reclaim_empty", "kvx_pool_compact_extent",
    "kvx_pool_snapshot_get", "kv_append", "kv_prepare_append", "kv_attend_decode_shared", "kvx_attend_shared_workspace_bytes", "kv_attend_verify", "kv_attend_verify_hidden", "kv_attend_decode",
    "kv_attend_prefill", "kv_attend_prefill_batch", "kv_compact_path", "kv_append_attend_decode", "kv_append_attend_decode_hidden", "kv_page_export", "kv_page_import", "kv_attend_split", "kv_attend_merge", "kv_attend_decode_static",
    "kvx_debug_attend_paths", "kvx_debug_prefill_tiles_together", "kvx_calibrate_stream", "kvx_decode_plan", "kvx_decode_plan_for", "kvx_prefill_plan_for", "kvx_verify_plan", "kvx_storage_create_accounting", "kvx_prefix_create", "kvx_prefix_destroy", "kvx_prefix_find",
    "kvx_prefix_insert", "kvx_prefix_contains", "kvx_prefix_generation", "kvx_prefix_block_count",
    "kvx_prefix_chain", "kvx_prefix_retain_active", "kvx_prefix_release_active",
    "kvx_prefix_touch", "kvx_prefix_eviction_candidate", "kvx_prefix_erase",
    "kvx_prefix_follow_pages", "kvx_prefix_match", "kvx_sequences_create",
    "kvx_sequences_destroy", "kvx_sequence_begin", "kvx_sequence_end", "kvx_sequence_restore",
    "kvx_sequence_ensure_tokens", "kvx_sequence_publish", "kvx_sequence_view",
    "kvx_sequences_compact_extent", "kvx_tree_masks", "kvx_tree_path_valid",
    "kvx_sequence_fork", "kvx_sequence_ensure_writable", "kvx_block_image_identity",
    "kvx_prefix_match_images", "kvx_sequence_publish_images", "kvx_sequence_truncate",
    "kvx_static_workspace_prime", "kvx_calibrate_stream_form",
]


class Layout(C.Structure):
    _fields_ = [("layers", C.c_uint32), ("kv_heads", C.c_uint32), ("head_dim", C.c_uint32),
                ("format", C.c_uint32), ("score_scale", C.c_float)]


class KvLayer(C.Structure):
    _fields_ = [("extent_pages", C.c_uint32), ("offset", C.c_uint32)]


class QkvShape(C.Structure):
    _fields_ = [("query_heads", C.c_uint32), ("rotary_pairs", C.c_uint32), ("query_gate", C.c_uint32),
                ("norm_type", C.c_uint32), ("eps", C.c_float)]


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


class SequencePages(C.Structure):
    _fields_ = [("pages", C.POINTER(C.c_uint32)), ("page_count", C.c_uint32),
                ("revision", C.c_uint64), ("first_changed", C.c_uint32),
                ("blocks", C.POINTER(C.c_uint64)), ("block_count", C.c_uint32)]


class PoolSnapshot(C.Structure):
    _fields_ = [("pages_allocated", C.c_uint32), ("pages_free", C.c_uint32),
                ("pages_active", C.c_uint32), ("pages_prefix", C.c_uint32),
                ("allocated_bytes", C.c_uint64), ("reclaimable_bytes", C.c_uint64),
                ("extent_allocations", C.c_uint64), ("extent_releases", C.c_uint64),
                ("extent_allocate_max_ms", C.c_double), ("extent_release_max_ms", C.c_double),
                ("extent_compactions", C.c_uint64), ("pages_moved", C.c_uint64)]


def _depends_on(child, parent):
    """The library objects behind `child` use those behind `parent` until they are destroyed,
    their destructors included, and the garbage collector may finalize a group of objects in
    any order: a parent closes the children that registered here before it closes itself.
    (Strong references: the collector clears weak ones before it runs any finalizer.)"""
    parent.__dict__.setdefault("_dependents", []).append(child)


def _close_dependents(parent):
    for child in reversed(parent.__dict__.pop("_dependents", [])):
        child.close()


class KvxError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"kvx error {code}: {message}")
        self.code = code


_lib = None


def lib():
    """Loads libkvx.so; raises when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m richengine_amd.build` "
                "(there is no CPU fallback for the KV path)")
        L = C.CDLL(LIB_PATH)
        _declare(L)
        _lib = L
    return _lib


def _declare(L):
    u32, u64, vp, i = C.c_uint32, C.c_uint64, C.c_void_p, C.c_int
    LP = C.POINTER(Layout)
    L.kvx_last_error.restype = C.c_char_p
    for n in ("kvx_layout_data_bytes_per_layer_page", "kvx_layout_scale_bytes_per_layer_page",
              "kvx_layout_bytes_per_layer_page", "kvx_layout_bytes_per_model_page"):
        getattr(L, n).argtypes, getattr(L, n).restype = [LP], u64
    for n in ("kvx_layout_extent_alignment_pages", "kvx_layout_minimum_extent_pages",
              "kvx_layout_maximum_extent_pages", "kvx_layout_largest_extent_pages"):
        getattr(L, n).argtypes, getattr(L, n).restype = [LP], u32
    L.kvx_layout_valid.argtypes = [LP]
    L.kvx_layout_extent_pages_for.argtypes, L.kvx_layout_extent_pages_for.restype = [LP, u64], u32
    L.kvx_kv_offset.argtypes, L.kvx_kv_offset.restype = [u32] * 6, u64
    for n in ("kvx_verify_splits", "kvx_decode_splits"):
        getattr(L, n).argtypes, getattr(L, n).restype = [u32, u32], u32
    L.kvx_prefill_splits.argtypes, L.kvx_prefill_splits.restype = [u32], u32
    L.kvx_prefill_plan.argtypes, L.kvx_prefill_plan.restype = [u32, u32, u32, u32, u32], u32
    L.kvx_prefill_plan_batch.argtypes, L.kvx_prefill_plan_batch.restype = [u32] * 6, u32
    L.kvx_chunk_validation.argtypes = [C.POINTER(ChunkParams)]
    P64 = C.POINTER(u64)
    L.kvx_prefill_workspace.argtypes = [u32, u32, LP, P64, P64]
    L.kvx_prefill_workspace_bound.argtypes = [u32, u32, LP, P64, P64]
    L.kvx_verify_workspace.argtypes = [u32, u32, u32, LP, P64, P64]
    L.kvx_attend_workspace_bytes.argtypes = [vp, u32, u32, LP]
    L.kvx_attend_workspace_bytes.restype = u64
    L.kvx_storage_create.argtypes = [LP, u32, u32, i, C.POINTER(vp)]
    L.kvx_storage_create_accounting.argtypes = [LP, u32, u32, i, C.POINTER(vp)]
    PU32, PU64 = C.POINTER(u32), C.POINTER(u64)
    L.kvx_prefix_create.argtypes = [vp, C.POINTER(vp)]
    L.kvx_prefix_destroy.argtypes, L.kvx_prefix_destroy.restype = [vp], None
    L.kvx_prefix_find.argtypes = [vp, u64, vp, u32, u64, u64, PU64, PU32]
    L.kvx_prefix_insert.argtypes = [vp, u64, vp, u32, u32, u64, u64, PU64, PU32]
    L.kvx_prefix_contains.argtypes = [vp, u64]
    L.kvx_prefix_generation.argtypes, L.kvx_prefix_generation.restype = [vp], u64
    L.kvx_prefix_block_count.argtypes, L.kvx_prefix_block_count.restype = [vp], u64
    L.kvx_prefix_chain.argtypes = [vp, u64, vp, vp, u32, PU32]
    for n in ("kvx_prefix_retain_active", "kvx_prefix_release_active", "kvx_prefix_touch",
              "kvx_prefix_erase"):
        getattr(L, n).argtypes = [vp, u64]
    L.kvx_prefix_eviction_candidate.argtypes = [vp, u64, PU64]
    L.kvx_prefix_follow_pages.argtypes, L.kvx_prefix_follow_pages.restype = [vp, u32, vp, u32], None
    L.kvx_prefix_match.argtypes, L.kvx_prefix_match.restype = [vp, vp, u64, vp, u32, PU32], u64
    L.kvx_sequences_create.argtypes = [vp, vp, C.POINTER(vp)]
    L.kvx_sequences_destroy.argtypes, L.kvx_sequences_destroy.restype = [vp], None
    L.kvx_sequence_begin.argtypes = [vp, u64]
    L.kvx_sequence_end.argtypes = [vp, u64]
    L.kvx_sequence_restore.argtypes = [vp, u64, u64]
    L.kvx_sequence_ensure_tokens.argtypes = [vp, u64, u64]
    L.kvx_sequence_publish.argtypes = [vp, u64, vp, u64, u32]
    L.kvx_sequence_view.argtypes = [vp, u64, C.POINTER(SequencePages)]
    L.kvx_sequences_compact_extent.argtypes = [vp, PU32, vp, PU32, vp]
    L.kvx_sequence_fork.argtypes = [vp, u64, u64, u64]
    L.kvx_sequence_ensure_writable.argtypes = [vp, u64, u64, PU32, PU32, PU32, vp]
    L.kvx_block_image_identity.argtypes = [u64, u32, vp, u32, PU64, PU64]
    L.kvx_block_image_identity.restype = None
    L.kvx_prefix_match_images.argtypes = [vp, vp, u64, vp, u32, vp, u32, PU32]
    L.kvx_prefix_match_images.restype = u64
    L.kvx_sequence_publish_images.argtypes = [vp, u64, vp, u64, u32, vp, u32]
    L.kvx_sequence_truncate.argtypes = [vp, u64, u64, PU32]
    L.kvx_debug_attend_paths.argtypes, L.kvx_debug_attend_paths.restype = [PU64, PU64], None
    L.kvx_debug_prefill_tiles_together.argtypes = [LP, u32, u32, u32, u32]
    L.kvx_debug_prefill_tiles_together.restype = u32
    L.kvx_calibrate_stream.argtypes = [vp, u32, vp, u32, u32, u32, vp, vp]
    L.kvx_calibrate_stream_form.argtypes = [vp, u32, vp, u32, u32, u32, u32, u32, vp, vp]
    L.kvx_decode_plan.argtypes = [vp, u32, u32, u32, vp]
    L.kvx_decode_plan_for.argtypes = [LP, vp, u32, vp]
    L.kvx_prefill_plan_for.argtypes, L.kvx_prefill_plan_for.restype = [LP, u32, u32, u32, u32], u32
    L.kvx_verify_plan.argtypes = [vp, u32, u32, u32, u32, u32, vp]
    L.kvx_tree_masks.argtypes = [vp, u32, vp]
    L.kvx_tree_path_valid.argtypes = [vp, u32, vp, u32]
    L.kvx_storage_destroy.argtypes = [vp]
    L.kvx_storage_destroy.restype = None
    for n in ("kvx_storage_page_count", "kvx_storage_extent_pages"):
        getattr(L, n).argtypes, getattr(L, n).restype = [vp], u32
    for n in ("kvx_storage_bytes_per_page", "kvx_storage_extent_bytes",
              "kvx_storage_allocated_bytes"):
        getattr(L, n).argtypes, getattr(L, n).restype = [vp], u64
    L.kvx_storage_is_allocated.argtypes = [vp, u32]
    L.kvx_storage_allocate_extent.argtypes = [vp, u32]
    L.kvx_storage_release_extent.argtypes = [vp, u32]
    L.kvx_storage_set_budget.argtypes, L.kvx_storage_set_budget.restype = [vp, u64], None
    L.kvx_storage_layer.argtypes = [vp, u32, C.POINTER(KvLayer)]
    L.kvx_storage_entries.argtypes = [vp, vp, u32, u32, vp]
    L.kvx_storage_write_entries.argtypes = [vp, vp, u32, u32, vp, u64, vp]
    L.kvx_storage_page_read.argtypes = [vp, u32, vp]
    L.kvx_storage_page_write.argtypes = [vp, u32, vp]
    L.kvx_storage_extent_read.argtypes = [vp, u32, u64, u64, vp]
    L.kvx_storage_extent_write.argtypes = [vp, u32, u64, u64, vp]
    L.kv_page_copy.argtypes = [vp, vp, u32, vp]
    L.kv_page_export.argtypes = [vp, vp, u32, vp, vp]
    L.kv_page_import.argtypes = [vp, vp, u32, vp, vp]
    L.kvx_pool_create.argtypes = [vp, u32, C.POINTER(vp)]
    L.kvx_pool_destroy.argtypes, L.kvx_pool_destroy.restype = [vp], None
    L.kvx_pool_acquire.argtypes = [vp, u32, vp]
    L.kvx_pool_retain.argtypes = [vp, u32, i]
    L.kvx_pool_release.argtypes = [vp, u32, i]
    L.kvx_pool_page_active.argtypes = [vp, u32]
    L.kvx_pool_free_pages.argtypes, L.kvx_pool_free_pages.restype = [vp], u32
    L.kvx_pool_reclaim_empty.argtypes = [vp, i, u32, P64]
    L.kvx_pool_compact_extent.argtypes = [vp, vp, u32, C.POINTER(u32), vp, C.POINTER(u32), vp]
    L.kvx_pool_snapshot_get.argtypes = [vp, C.POINTER(PoolSnapshot)]
    L.kv_append.argtypes = [vp, u32, vp, vp, vp, vp, u32, u64, u32, vp]
    L.kv_prepare_append.argtypes = [vp, u32, C.POINTER(QkvShape), vp, vp, vp, vp, vp, vp, u32, vp, vp,
                                    u32, u32, u32, vp]
    L.kv_attend_verify.argtypes = [vp, u32, u32, vp, vp, vp, vp, u32, vp, u32, vp, u64, vp]
    L.kv_attend_verify_hidden.argtypes = [vp, u32, u32, vp, vp, vp, vp, u32, vp, u32, vp, u64, vp, vp,
                                          vp]
    L.kv_attend_decode.argtypes = [vp, u32, u32, vp, vp, vp, vp, u32, u32, vp, u64, vp]
    L.kv_attend_decode_static.argtypes = [vp, u32, u32, vp, vp, vp, vp, u32, u32, vp]
    L.kv_attend_split.argtypes = [vp, u32, u32, vp, vp, vp, u32, vp, u32, vp, u64, vp]
    L.kv_attend_merge.argtypes = [vp, u32, vp, vp, u32, u32, vp, u64, vp]
    L.kv_attend_decode_shared.argtypes = [vp, u32, u32, vp, vp, vp, vp, u32, u32, u32, u32, vp, u64, vp]
    L.kvx_attend_shared_workspace_bytes.argtypes = [vp, u32, u32, u32, C.POINTER(Layout)]
    L.kvx_attend_shared_workspace_bytes.restype = u64
    L.kv_append_attend_decode.argtypes = [vp, u32, vp, vp, u64, u32, u32, vp, vp, vp, vp, u32, u32, vp,
                                          u64, vp]
    L.kv_append_attend_decode_hidden.argtypes = [vp, u32, vp, vp, u64, u32, u32, vp, vp, vp, vp, u32, u32,
                                                 vp, u64, vp, vp, vp]
    L.kv_attend_prefill.argtypes = [vp, u32, u32, vp, vp, vp, C.POINTER(PrefillParams), vp, u64, vp]
    L.kv_attend_prefill_batch.argtypes = [vp, u32, u32, vp, vp, vp, C.POINTER(PrefillParams), u32, u64, vp, u64, vp]
    L.kv_compact_path.argtypes = [vp, u32, vp, vp, u32, vp, vp, u32, vp]


def check(rc):
    if rc != OK:
        raise KvxError(rc, lib().kvx_last_error().decode())
    return rc


def _stream(stream):
    if stream is not None:
        return C.c_void_p(stream or None)  # 0 = the default stream
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    """Device address of a torch tensor (or an int / None)."""
    if t is None:
        return None
    return t if isinstance(t, int) else t.data_ptr()


def _table_array(tables):
    return (C.c_void_p * len(tables))(*[_ptr(t) for t in tables])


class Storage:
    """Page storage in device extents (the reference's kv::PageStorage)."""

    def __init__(self, layers, kv_heads, head_dim, fmt, page_count, extent_pages, aligned=False,
                 score_scale=0.0, accounting=False):
        self.layout = Layout(layers, kv_heads, head_dim, fmt, score_scale)
        self.accounting = accounting
        h = C.c_void_p()
        create = lib().kvx_storage_create_accounting if accounting else lib().kvx_storage_create
        check(create(C.byref(self.layout), page_count, extent_pages, int(aligned), C.byref(h)))
        self.h = h
        self.page_count, self.extent_pages = page_count, extent_pages
        self.extents = page_count // extent_pages
        self.extent_bytes = lib().kvx_storage_extent_bytes(h)
        self.bytes_per_page = lib().kvx_storage_bytes_per_page(h)

    def close(self):
        _close_dependents(self)
        if getattr(self, "h", None):
            lib().kvx_storage_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except TypeError:   # the interpreter is shutting down and this module's names are gone
            pass

    def allocate(self, extent):
        return check(lib().kvx_storage_allocate_extent(self.h, extent))

    def allocate_all(self):
        for e in range(self.extents):
            self.allocate(e)
        return self

    def release(self, extent):
        return check(lib().kvx_storage_release_extent(self.h, extent))

    def layer(self, layer):
        out = KvLayer()
        check(lib().kvx_storage_layer(self.h, layer, C.byref(out)))
        return out

    def entries_host(self, pages, first=0):
        import numpy as np
        pages = np.ascontiguousarray(pages, dtype=np.uint32)
        table = np.zeros(len(pages), dtype=np.uint64)
        check(lib().kvx_storage_entries(self.h, pages.ctypes.data, len(pages), first,
                                        table.ctypes.data))
        return table

    def table(self, pages):
        """A device page table (torch int64 tensor holding the u64 entries)."""
        import torch
        host = self.entries_host(pages)
        return torch.from_numpy(host.view("int64")).cuda()

    def page_read(self, page):
        import numpy as np
        out = np.empty(self.bytes_per_page, dtype=np.uint8)
        check(lib().kvx_storage_page_read(self.h, page, out.ctypes.data))
        return out

    def page_write(self, page, data):
        import numpy as np
        data = np.ascontiguousarray(data, dtype=np.uint8)
        assert data.size == self.bytes_per_page
        return check(lib().kvx_storage_page_write(self.h, page, data.ctypes.data))

    def extent_read(self, extent, offset=0, nbytes=None):
        import numpy as np
        nbytes = self.extent_bytes - offset if nbytes is None else nbytes
        out = np.empty(nbytes, dtype=np.uint8)
        check(lib().kvx_storage_extent_read(self.h, extent, offset, nbytes, out.ctypes.data))
        return out

    def extent_write(self, extent, data, offset=0):
        import numpy as np
        data = np.ascontiguousarray(data, dtype=np.uint8)
        return check(lib().kvx_storage_extent_write(self.h, extent, offset, data.size,
                                                    data.ctypes.data))

    def export_pages(self, pages, buffer, stream=None):
        """Wire bytes of `pages` into `buffer` (device or pinned host tensor)."""
        return check(lib().kv_page_export(self.h, _u32(pages), len(pages), _ptr(buffer), _stream(stream)))

    def import_pages(self, pages, buffer, stream=None):
        return check(lib().kv_page_import(self.h, _u32(pages), len(pages), _ptr(buffer), _stream(stream)))

    def copy_pages(self, copies, stream=None):
        arr = (PageCopy * len(copies))(*[PageCopy(a, b) for a, b in copies])
        return check(lib().kv_page_copy(self.h, arr, len(copies), _stream(stream)))


def append(storage, layer, chunk_keys, chunk_values, tables, lanes, lane_stride,
           verify_max_rows=0, stream=None):
    arr = (ChunkParams * len(lanes))(*lanes)
    return check(lib().kv_append(storage.h, layer, _ptr(chunk_keys), _ptr(chunk_values),
                                 _table_array(tables), arr, len(lanes), lane_stride,
                                 verify_max_rows, _stream(stream)))


def attend_workspace_bytes(storage, lanes, query_heads):
    arr = (VerifyParams * len(lanes))(*lanes)
    return lib().kvx_attend_workspace_bytes(arr, len(lanes), query_heads, C.byref(storage.layout))


def prepare_append(storage, layer, shape, packed_qkv, q_norm, k_norm, rope_cos, rope_sin, queries,
                   row_stride, tables, lanes, rows, verify_max_rows=0, stream=None):
    """QKV prepare fused with quantize-on-append (kv_prepare_append)."""
    arr = (ChunkParams * len(lanes))(*lanes)
    return check(lib().kv_prepare_append(storage.h, layer, C.byref(shape), _ptr(packed_qkv),
                                         _ptr(q_norm), _ptr(k_norm), _ptr(rope_cos), _ptr(rope_sin),
                                         _ptr(queries), row_stride, _table_array(tables), arr,
                                         len(lanes), rows, verify_max_rows, _stream(stream)))


def attend_verify(storage, layer, query_heads, queries, output, tables, lanes, row_masks,
                  row_stride, workspace, stream=None):
    arr = (VerifyParams * len(lanes))(*lanes)
    return check(lib().kv_attend_verify(storage.h, layer, query_heads, _ptr(queries), _ptr(output),
                                        _table_array(tables), arr, len(lanes), _ptr(row_masks),
                                        row_stride, _ptr(workspace),
                                        workspace.numel() * workspace.element_size(),
                                        _stream(stream)))


def attend_split(storage, layer, query_heads, queries, tables, lanes, row_masks, row_stride,
                 workspace, stream=None):
    """The split dispatch alone: partial rows and statistics of every split into `workspace`."""
    arr = lanes if isinstance(lanes, C.Array) else (VerifyParams * len(lanes))(*lanes)
    return check(lib().kv_attend_split(storage.h, layer, query_heads, _ptr(queries),
                                       _table_array(tables), arr, len(arr), _ptr(row_masks),
                                       row_stride, _ptr(workspace),
                                       workspace.numel() * workspace.element_size(), _stream(stream)))


def attend_merge(storage, query_heads, output, lanes, row_stride, workspace, stream=None):
    """The merge dispatch alone over a workspace in kv_attend_split's layout."""
    arr = lanes if isinstance(lanes, C.Array) else (VerifyParams * len(lanes))(*lanes)
    return check(lib().kv_attend_merge(storage.h, query_heads, _ptr(output), arr, len(arr),
                                       row_stride, _ptr(workspace),
                                       workspace.numel() * workspace.element_size(), _stream(stream)))


def attend_verify_hidden(storage, layer, query_heads, queries, output, tables, lanes, row_masks,
                         row_stride, workspace, packed_qkv, hidden, stream=None):
    """attend_verify whose merge also writes the out-projection's operand `hidden`
    ([lane][row capacity][query head][D]), gated by `packed_qkv` when that is given; `output`
    may be None."""
    arr = (VerifyParams * len(lanes))(*lanes)
    return check(lib().kv_attend_verify_hidden(
        storage.h, layer, query_heads, _ptr(queries), _ptr(output), _table_array(tables), arr,
        len(lanes), _ptr(row_masks), row_stride, _ptr(workspace),
        workspace.numel() * workspace.element_size(), _ptr(packed_qkv), _ptr(hidden),
        _stream(stream)))


def attend_decode(storage, layer, query_heads, queries, output, tables, lanes, row_stride,
                  workspace, stream=None):
    arr = (VerifyParams * len(lanes))(*lanes)
    return check(lib().kv_attend_decode(storage.h, layer, query_heads, _ptr(queries), _ptr(output),
                                        _table_array(tables), arr, len(lanes), row_stride,
                                        _ptr(workspace),
                                        workspace.numel() * workspace.element_size(),
                                        _stream(stream)))


def attend_decode_static(storage, layer, query_heads, queries, output, tables, lanes, row_stride,
                         stream=None):
    """kv_attend_decode over the library's static workspace (kv_attend_decode_static)."""
    arr = (VerifyParams * len(lanes))(*lanes)
    return check(lib().kv_attend_decode_static(storage.h, layer, query_heads, _ptr(queries),
                                               _ptr(output), _table_array(tables), arr, len(lanes),
                                               row_stride, _stream(stream)))


def attend_shared_workspace_bytes(storage, lanes, prefix_splits, query_heads):
    arr = (VerifyParams * len(lanes))(*lanes)
    return lib().kvx_attend_shared_workspace_bytes(arr, len(lanes), prefix_splits, query_heads,
                                                   C.byref(storage.layout))


def attend_decode_shared(storage, layer, query_heads, queries, output, tables, lanes, shared_pages,
                         prefix_splits, row_stride, workspace, stream=None):
    """One-row decode of sequences whose tables begin with the same `shared_pages` pages."""
    arr = (VerifyParams * len(lanes))(*lanes)
    return check(lib().kv_attend_decode_shared(
        storage.h, layer, query_heads, _ptr(queries), _ptr(output), _table_array(tables), arr,
        len(lanes), shared_pages, prefix_splits, row_stride, _ptr(workspace),
        workspace.numel() * workspace.element_size(), _stream(stream)))


def append_attend_decode(storage, layer, chunk_keys, chunk_values, chunk_lane_stride, chunk_stride,
                         query_heads, queries, output, tables, lanes, row_stride, workspace,
                         stream=None):
    arr = (VerifyParams * len(lanes))(*lanes)
    return check(lib().kv_append_attend_decode(
        storage.h, layer, _ptr(chunk_keys), _ptr(chunk_values), chunk_lane_stride, chunk_stride,
        query_heads, _ptr(queries), _ptr(output), _table_array(tables), arr, len(lanes), row_stride,
        _ptr(workspace), workspace.numel() * workspace.element_size(), _stream(stream)))


def append_attend_decode_hidden(storage, layer, chunk_keys, chunk_values, chunk_lane_stride,
                                chunk_stride, query_heads, queries, output, tables, lanes, row_stride,
                                workspace, packed_qkv, hidden, stream=None):
    """append_attend_decode whose merge also writes the out-projection's operand `hidden`, gated by
    `packed_qkv` when that is given; `output` may be None."""
    arr = (VerifyParams * len(lanes))(*lanes)
    return check(lib().kv_append_attend_decode_hidden(
        storage.h, layer, _ptr(chunk_keys), _ptr(chunk_values), chunk_lane_stride, chunk_stride,
        query_heads, _ptr(queries), _ptr(output), _table_array(tables), arr, len(lanes), row_stride,
        _ptr(workspace), workspace.numel() * workspace.element_size(), _ptr(packed_qkv), _ptr(hidden),
        _stream(stream)))


def prefill_workspace_bytes(storage, rows, query_heads, splits=None):
    """Workspace of kv_attend_prefill: for the reference's split rule, or for `splits`."""
    pb, sb = C.c_uint64(), C.c_uint64()
    if splits is None:
        check(lib().kvx_prefill_workspace(rows, query_heads, C.byref(storage.layout), C.byref(pb),
                                          C.byref(sb)))
    else:
        check(lib().kvx_prefill_workspace_for(rows, splits, query_heads, C.byref(storage.layout),
                                              C.byref(pb), C.byref(sb)))
    return pb.value + sb.value


def attend_prefill(storage, layer, query_heads, queries, output, table, params, workspace,
                   stream=None):
    return check(lib().kv_attend_prefill(storage.h, layer, query_heads, _ptr(queries),
                                         _ptr(output), _ptr(table), C.byref(params),
                                         _ptr(workspace),
                                         workspace.numel() * workspace.element_size(),
                                         _stream(stream)))


def attend_prefill_batch(storage, layer, query_heads, queries, output, tables, params,
                         sequence_stride, workspace, stream=None):
    """The chunks of several sequences in one call: sequence q's queries and rows begin
    q x sequence_stride elements after the first's."""
    arr = (PrefillParams * len(params))(*params)
    return check(lib().kv_attend_prefill_batch(
        storage.h, layer, query_heads, _ptr(queries), _ptr(output), _table_array(tables), arr,
        len(params), sequence_stride, _ptr(workspace),
        workspace.numel() * workspace.element_size(), _stream(stream)))


def compact_path(storage, layer, tables, lanes, retained_path, retained_count, path_stride,
                 stream=None):
    arr = (ChunkParams * len(lanes))(*lanes)
    return check(lib().kv_compact_path(storage.h, layer, _table_array(tables), arr, len(lanes),
                                       _ptr(retained_path), _ptr(retained_count), path_stride,
                                       _stream(stream)))


class Pool:
    """Page references and extent lifetime (the reference's engine::KvPool)."""

    def __init__(self, storage, runway_pages):
        h = C.c_void_p()
        check(lib().kvx_pool_create(storage.h, runway_pages, C.byref(h)))
        self.h, self.storage = h, storage
        _depends_on(self, storage)

    def close(self):
        _close_dependents(self)
        if getattr(self, "h", None):
            lib().kvx_pool_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except TypeError:   # the interpreter is shutting down and this module's names are gone
            pass

    def acquire(self, count):
        out = (C.c_uint32 * max(count, 1))()
        check(lib().kvx_pool_acquire(self.h, count, out))
        return list(out[:count])

    def retain(self, page, prefix_owner=False):
        return check(lib().kvx_pool_retain(self.h, page, int(prefix_owner)))

    def release(self, page, prefix_owner=False):
        return check(lib().kvx_pool_release(self.h, page, int(prefix_owner)))

    def page_active(self, page):
        return bool(lib().kvx_pool_page_active(self.h, page))

    def reclaim_empty(self, keep_runway, limit=0xFFFFFFFF):
        out = C.c_uint64()
        check(lib().kvx_pool_reclaim_empty(self.h, int(keep_runway), limit, C.byref(out)))
        return out.value

    def compact_extent(self, fixed=(), stream=None):
        fixed_arr = (C.c_uint32 * max(len(fixed), 1))(*fixed)
        first, moved = C.c_uint32(), C.c_uint32()
        dest = (C.c_uint32 * self.storage.extent_pages)()
        if stream is None and self.storage.accounting:
            stream = 0
        check(lib().kvx_pool_compact_extent(self.h, fixed_arr, len(fixed), C.byref(first), dest,
                                            C.byref(moved), _stream(stream)))
        if not moved.value:
            return None
        return {"first": first.value, "dest": list(dest), "moved": moved.value}

    def snapshot(self):
        s = PoolSnapshot()
        check(lib().kvx_pool_snapshot_get(self.h, C.byref(s)))
        return s


def _u32(values):
    return (C.c_uint32 * max(len(values), 1))(*[int(v) for v in values])


class Prefix:
    """Prefix page cache, resident tier (the reference's engine::KvCache)."""

    def __init__(self, pool):
        h = C.c_void_p()
        check(lib().kvx_prefix_create(pool.h, C.byref(h)))
        self.h, self.pool = h, pool
        _depends_on(self, pool)

    def close(self):
        _close_dependents(self)
        if getattr(self, "h", None):
            lib().kvx_prefix_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except TypeError:   # the interpreter is shutting down and this module's names are gone
            pass

    def find(self, parent, tokens, images=(0, 0)):
        block, page = C.c_uint64(), C.c_uint32()
        found = lib().kvx_prefix_find(self.h, parent, _u32(tokens), len(tokens), images[0],
                                      images[1], C.byref(block), C.byref(page))
        return (block.value, page.value) if found else None

    def insert(self, parent, tokens, page, images=(0, 0)):
        block, canonical = C.c_uint64(), C.c_uint32()
        check(lib().kvx_prefix_insert(self.h, parent, _u32(tokens), len(tokens), page, images[0],
                                      images[1], C.byref(block), C.byref(canonical)))
        return block.value, canonical.value

    def contains(self, block):
        return bool(lib().kvx_prefix_contains(self.h, block))

    def generation(self):
        return lib().kvx_prefix_generation(self.h)

    def block_count(self):
        return lib().kvx_prefix_block_count(self.h)

    def chain(self, block):
        length = C.c_uint32()
        check(lib().kvx_prefix_chain(self.h, block, None, None, 0, C.byref(length)))
        blocks, pages = (C.c_uint64 * max(length.value, 1))(), (C.c_uint32 * max(length.value, 1))()
        check(lib().kvx_prefix_chain(self.h, block, blocks, pages, length.value, C.byref(length)))
        return list(blocks[:length.value]), list(pages[:length.value])

    def retain_active(self, block):
        return check(lib().kvx_prefix_retain_active(self.h, block))

    def release_active(self, block):
        return check(lib().kvx_prefix_release_active(self.h, block))

    def touch(self, block):
        return check(lib().kvx_prefix_touch(self.h, block))

    def eviction_candidate(self, after=0):
        block = C.c_uint64()
        rc = lib().kvx_prefix_eviction_candidate(self.h, after, C.byref(block))
        if rc < 0:
            check(rc)
        return block.value if rc else None

    def erase(self, block):
        return check(lib().kvx_prefix_erase(self.h, block))

    def follow_pages(self, moves):
        if moves:
            dest = _u32(moves["dest"])
            lib().kvx_prefix_follow_pages(self.h, moves["first"], dest, len(moves["dest"]))

    def match(self, prompt, spans=()):
        """spans: the prompt's images as (offset, tokens, grid height, grid width, digest lo,
        digest hi) tuples sorted by offset; none for a text-only prompt."""
        capacity = max(len(prompt) // 32, 1)
        blocks, matched = (C.c_uint64 * capacity)(), C.c_uint32()
        if spans:
            arr = (ImageSpan * len(spans))(*[ImageSpan(*s) for s in spans])
            hashed = lib().kvx_prefix_match_images(self.h, _u32(prompt), len(prompt), arr, len(spans),
                                                   blocks, capacity, C.byref(matched))
        else:
            hashed = lib().kvx_prefix_match(self.h, _u32(prompt), len(prompt), blocks, capacity,
                                            C.byref(matched))
        return list(blocks[:matched.value]), hashed


class Sequences:
    """Per-sequence page lists (the Request records of the reference's engine::Cache)."""

    def __init__(self, pool, prefix):
        h = C.c_void_p()
        check(lib().kvx_sequences_create(pool.h, prefix.h, C.byref(h)))
        self.h, self.pool, self.prefix = h, pool, prefix
        _depends_on(self, prefix)

    def close(self):
        if getattr(self, "h", None):
            lib().kvx_sequences_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except TypeError:   # the interpreter is shutting down and this module's names are gone
            pass

    def begin(self, sequence):
        return check(lib().kvx_sequence_begin(self.h, sequence))

    def end(self, sequence):
        return check(lib().kvx_sequence_end(self.h, sequence))

    def restore(self, sequence, last_block):
        return check(lib().kvx_sequence_restore(self.h, sequence, last_block))

    def ensure_tokens(self, sequence, tokens):
        return check(lib().kvx_sequence_ensure_tokens(self.h, sequence, tokens))

    def publish(self, sequence, tokens, committed, spans=()):
        if spans:
            arr = (ImageSpan * len(spans))(*[ImageSpan(*s) for s in spans])
            return check(lib().kvx_sequence_publish_images(self.h, sequence, _u32(tokens), len(tokens),
                                                           committed, arr, len(spans)))
        return check(lib().kvx_sequence_publish(self.h, sequence, _u32(tokens), len(tokens),
                                                committed))

    def truncate(self, sequence, tokens):
        """Gives back the pages past those of the first `tokens` tokens; returns how many."""
        released = C.c_uint32()
        check(lib().kvx_sequence_truncate(self.h, sequence, tokens, C.byref(released)))
        return released.value

    def fork(self, sequence, source, tokens):
        """`sequence` (empty) shares the pages of the first `tokens` tokens of `source`."""
        return check(lib().kvx_sequence_fork(self.h, sequence, source, tokens))

    def ensure_writable(self, sequence, token, stream=None):
        """Copy-on-write of the page that holds `token`: None when the page is written in
        place, else (shared page, the sequence's new copy)."""
        if stream is None and self.pool.storage.accounting:
            stream = 0
        copied, source, copy = C.c_uint32(), C.c_uint32(), C.c_uint32()
        check(lib().kvx_sequence_ensure_writable(self.h, sequence, token, C.byref(copied),
                                                 C.byref(source), C.byref(copy), _stream(stream)))
        return (source.value, copy.value) if copied.value else None

    def view(self, sequence):
        out = SequencePages()
        check(lib().kvx_sequence_view(self.h, sequence, C.byref(out)))
        return {"pages": [out.pages[i] for i in range(out.page_count)],
                "revision": out.revision, "first_changed": out.first_changed,
                "blocks": [out.blocks[i] for i in range(out.block_count)]}

    def compact_extent(self, stream=None):
        if stream is None and self.pool.storage.accounting:
            stream = 0
        first, moved = C.c_uint32(), C.c_uint32()
        dest = (C.c_uint32 * self.pool.storage.extent_pages)()
        check(lib().kvx_sequences_compact_extent(self.h, C.byref(first), dest, C.byref(moved),
                                                 _stream(stream)))
        if not moved.value:
            return None
        return {"first": first.value, "dest": list(dest), "moved": moved.value}


class ImageSpan(C.Structure):
    _fields_ = [("offset", C.c_uint32), ("tokens", C.c_uint32), ("grid_height", C.c_uint32),
                ("grid_width", C.c_uint32), ("digest_lo", C.c_uint64), ("digest_hi", C.c_uint64)]


def block_image_identity(block_begin, block_tokens, spans):
    """(lo, hi) of the images overlapping a block; spans = (offset, tokens, grid height, grid
    width, digest lo, digest hi) tuples sorted by offset (kvx_block_image_identity)."""
    arr = (ImageSpan * max(len(spans), 1))(*[ImageSpan(*s) for s in spans])
    lo, hi = C.c_uint64(), C.c_uint64()
    lib().kvx_block_image_identity(block_begin, block_tokens, arr, len(spans), C.byref(lo), C.byref(hi))
    return lo.value, hi.value


def decode_plan(committed, kv_heads, fmt=INT4):
    """Split counts of a decode batch of pages of format `fmt` (kvx_decode_plan)."""
    out = (C.c_uint32 * len(committed))()
    check(lib().kvx_decode_plan(_u32(committed), len(committed), kv_heads, fmt, out))
    return list(out)


def decode_plan_for(storage, committed):
    """Split counts of a decode batch sized for the GPU and the storage's layout (kvx_decode_plan_for)."""
    out = (C.c_uint32 * len(committed))()
    check(lib().kvx_decode_plan_for(C.byref(storage.layout), _u32(committed), len(committed), out))
    return list(out)


def prefill_plan_for(storage, committed, rows, query_heads, sequences=1):
    """Split count of a chunked prefill sized for the GPU and the storage's layout (kvx_prefill_plan_for)."""
    splits = lib().kvx_prefill_plan_for(C.byref(storage.layout), committed, rows, query_heads, sequences)
    if not splits:
        raise KvxError(-1, "kvx_prefill_plan_for: bad layout or head counts")
    return splits


def prefill_plan(committed, rows, kv_heads, query_heads, fmt=INT4, sequences=1):
    """Split count of a chunked prefill sized for the GPU (kvx_prefill_plan; for `sequences`
    equal chunks in one kv_attend_prefill_batch call, kvx_prefill_plan_batch)."""
    splits = lib().kvx_prefill_plan_batch(committed, rows, kv_heads, query_heads, fmt, sequences)
    if not splits:
        raise KvxError(-1, "kvx_prefill_plan: bad head counts")
    return splits


def verify_plan(committed, rows, kv_heads, query_heads, fmt=INT4):
    """Split counts of a verify batch sized for the GPU (kvx_verify_plan)."""
    out = (C.c_uint32 * len(committed))()
    check(lib().kvx_verify_plan(_u32(committed), len(committed), rows, kv_heads, query_heads, fmt, out))
    return list(out)


def attend_paths():
    """(generic, matrix-core) attend call counts of this process."""
    generic, matrix = C.c_uint64(), C.c_uint64()
    lib().kvx_debug_attend_paths(C.byref(generic), C.byref(matrix))
    return generic.value, matrix.value


def tree_masks(parents):
    masks = (C.c_uint32 * max(len(parents), 1))()
    check(lib().kvx_tree_masks(_u32(parents), len(parents), masks))
    return list(masks[:len(parents)])


def tree_path_valid(parents, path):
    return bool(lib().kvx_tree_path_valid(_u32(parents), len(parents), _u32(path), len(path)))
