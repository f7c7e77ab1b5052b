"""Shared fixtures of the GPU parity tests: twin pools (oracle on the host, the
library on the device) with the same geometry and page ids, and comparisons."""
import ctypes as C

import numpy as np
import torch

from oracle import kvoracle as ko
from richengine_amd import kvx
import kvtestlib as T


def dev(a):
    """numpy array -> device tensor with the same bytes (uint16 travels as int16)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16)).cuda()
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32)).cuda()
    if a.dtype == np.uint64:
        return torch.from_numpy(a.view(np.int64)).cuda()
    return torch.from_numpy(a).cuda()


def host_u16(t):
    return t.cpu().numpy().view(np.uint16)


class Twin:
    """An oracle store and a device storage of identical geometry."""

    def __init__(self, fmt, kv_heads, head_dim, layers, pages_needed, one_extent=False):
        ep, n = T.spread(pages_needed + 2)
        if one_extent:
            ep, n = ep * n, 1
        self.fmt, self.H, self.D, self.layers = fmt, kv_heads, head_dim, layers
        self.host = ko.Store(layers, kv_heads, head_dim, fmt, ep * n, ep)
        self.dev = kvx.Storage(layers, kv_heads, head_dim, fmt, ep * n, ep)
        for e in range(n):
            assert self.host.allocate(e) == 0
            self.dev.allocate(e)
        self.extent_pages, self.extents = ep, n

    def pages(self, count, seed):
        return T.mixed_pages(self.extent_pages, self.extents, count, seed)

    def tables(self, pages):
        return self.host.entries(pages), self.dev.table(pages)

    def assert_same_bytes(self):
        for e in range(self.extents):
            got = self.dev.extent_read(e)
            want = self.host.extent(e)
            if not np.array_equal(got, want):
                bad = np.flatnonzero(got != want)
                raise AssertionError(f"extent {e}: {bad.size} bytes differ, first at {bad[0]}: "
                                     f"got {got[bad[0]]:#x} want {want[bad[0]]:#x}")

    def download(self):
        """Copies the device extents' bytes into the oracle store (after device
        appends whose bit-exactness other tests pin)."""
        for e in range(self.extents):
            self.host.extent(e)[:] = self.dev.extent_read(e)

    def upload(self):
        """Copies the oracle store's bytes into the device extents."""
        for e in range(self.extents):
            self.dev.extent_write(e, self.host.extent(e))

    def close(self):
        self.dev.close()
        self.host.close()


def ko_chunk(p, layer_obj):
    return ko.ChunkParams(p.committed_tokens, p.chunk_tokens, p.chunk_stride, p.page_table_entries,
                          ko.KvLayer(layer_obj.extent_pages, layer_obj.offset))


def bf16_ulp_diff(a_bits, b_bits):
    """Distance in bf16 codes between two uint16 arrays (sign-magnitude aware)."""
    def key(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7FFF), x & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


def check_attention(out_bits, want_bits, want_f32, rows_mask, tol, label="", matrix_core=False):
    """out_bits / want_bits: bf16 outputs (GPU, oracle); want_f32: the oracle's
    value before its final rounding.  rows_mask selects live rows (last axis D).

    Bar, per output row: ||gpu - oracle||2 / ||oracle||2 <= tol on the bf16
    outputs both sides produce.  Against the oracle's fp32 value the bound is
    tol + 2e-3, because rounding a row to bf16 alone moves it by 1.6e-3 to
    2.0e-3 in this norm (the oracle's own bf16 output is that far from its
    fp32 value), which would leave no room for anything else.

    matrix_core: kernels that sum q.k on the matrix cores cannot keep the
    oracle's summation order, so a score can differ in its last bits and the
    bf16 rounding of one probability can fall the other way.  When that
    probability dominates its row, the row moves by up to half a bf16 step
    (2e-3) on top of everything else.  For those kernels at least 99% of the
    rows must meet tol and every row tol + 2e-3."""
    got = ko.bf16_to_f32(out_bits).reshape(out_bits.shape)
    want = ko.bf16_to_f32(want_bits).reshape(want_bits.shape)
    assert np.isfinite(got).all(), f"{label}: non-finite attention output"
    rel = T.rel_l2(got[rows_mask], want[rows_mask])
    flat = np.unravel_index(int(np.argmax(rel)), rel.shape)
    worst = tuple(int(x) for x in np.argwhere(rows_mask)[flat[0]]) + tuple(int(x) for x in flat[1:])
    hard = tol + 2e-3 if matrix_core else tol
    assert rel.max() <= hard, (f"{label}: relative L2 vs oracle bf16 {rel.max():.3e} > {hard} "
                               f"at row {worst}")
    within = float((rel <= tol).mean())
    # 1% of the rows, and at least one where there are fewer than a hundred
    allowed = max(1, int(0.01 * rel.size)) if matrix_core else 0
    assert int((rel > tol).sum()) <= allowed, (
        f"{label}: only {within:.4f} of the {rel.size} rows are within {tol}")
    rel32 = T.rel_l2(got[rows_mask], want_f32[rows_mask])
    assert rel32.max() <= tol + 2e-3, f"{label}: relative L2 vs oracle fp32 {rel32.max():.3e}"
    ulps = bf16_ulp_diff(out_bits[rows_mask], want_bits[rows_mask])
    return dict(rel_l2=float(rel.max()), rel_l2_mean=float(rel.mean()), rows_within_tol=within,
                rel_l2_fp32=float(rel32.max()),
                max_abs=float(np.abs(got[rows_mask] - want_f32[rows_mask]).max()),
                exact=float((ulps == 0).mean()), max_ulp=int(ulps.max()))


def oracle_tile(fmt, kv_heads, group, head_dim, tile_queries, table, kv, head, committed, active,
                splits, capacity, masks=None, score_scale=0.0):
    """The oracle's attention of one tile (capacity rows x group fused rows) of one
    KV head: every split's partial tile, then the fixed-order merge of each live
    fused row.  tile_queries: bf16 [capacity * group, D].  Returns (bf16, fp32)
    outputs of that shape; rows past `active` are zeros."""
    L = ko.lib()
    M, D = capacity * group, head_dim
    tile_queries = np.ascontiguousarray(tile_queries, dtype=np.uint16).reshape(M, D)
    partials = np.zeros((splits, M, D), dtype=np.float32)
    statistics = np.zeros((splits, M, 2), dtype=np.float32)
    mask_ptr = ko.ptr(np.ascontiguousarray(masks, dtype=np.uint32)) if masks is not None else None
    for split in range(splits):
        L.ko_attention_tile(fmt, kv_heads, group, D, capacity, ko.ptr(tile_queries), ko.ptr(table), kv,
                            head, committed, active, splits, split, ko.ptr(partials),
                            ko.ptr(statistics), split, mask_ptr, score_scale)
    out = np.zeros((M, D), dtype=np.uint16)
    out32 = np.zeros((M, D), dtype=np.float32)
    for row in range(M):
        L.ko_attention_reduce_row(group, D, capacity, ko.ptr(partials), ko.ptr(statistics), committed,
                                  active, splits, 0, row, ko.ptr(out[row]), ko.ptr(out32[row]))
    return out, out32
