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


# Rows that were farther from the oracle than the tolerance and were shown to be one
# rounding flip away from it, per check: (label, rows explained, rows checked).
ALLOWANCE_LOG = []
# What tests/test_gpu_score_deviation.py measured, per format: (name, samples, worst |max - max|,
# worst |max + log(sum) - the same|, the flip slack the format's checks use).
DEVIATION_LOG = []


def check_attention(out_bits, want_bits, want_f32, rows_mask, tol, label="", explain=None):
    """out_bits / want_bits: bf16 outputs (GPU, oracle); want_f32: the oracle's
    value before its final rounding.  rows_mask selects live rows (last axis D).

    Bar, per output row: ||gpu - oracle||2 / ||oracle||2 <= tol on the bf16
    outputs both sides produce.  Against the oracle's fp32 value the bound is
    tol + 2e-3, because rounding a row to bf16 alone moves it by 1.6e-3 to
    2.0e-3 in this norm (the oracle's own bf16 output is that far from its
    fp32 value), which would leave no room for anything else.

    explain: for kernels that sum q.k on the matrix cores, which cannot keep the
    oracle's summation order: a score can differ in its last bits, so the rounding
    of one probability (to bf16; fp16 on fp8 pages) can fall the other way, and when
    that token carries most of its row the row moves by up to half a place.  A row
    above tol is accepted only if that is shown to be what happened: explain(index)
    describes the row's tile (keyword arguments of ko.rounding_flip_rows, or {"rows": ...}
    with such rows from an arrangement of the caller's own), the oracle
    recomputes the row with the rounded weight of one of its heaviest tokens moved
    one place up or down, and one of those rows must be within tol of the GPU's.
    At most 1% of the rows (two where there are fewer than two hundred) may need it and
    none may be more than tol + 2^-7 away (one place of a weight just above a power of
    two, were the row that one token); every such row is counted in ALLOWANCE_LOG."""
    got = ko.bf16_to_f32(out_bits).reshape(out_bits.shape)
    want = ko.bf16_to_f32(want_bits).reshape(want_bits.shape)
    assert np.isfinite(got).all(), f"{label}: non-finite attention output"
    rel = T.rel_l2(got[rows_mask], want[rows_mask])
    coords = np.argwhere(rows_mask)

    def index_of(flat):
        at = np.unravel_index(int(flat), rel.shape)
        return tuple(int(x) for x in coords[at[0]]) + tuple(int(x) for x in at[1:])

    over = np.flatnonzero(rel.ravel() > tol)
    within = 1.0 - over.size / rel.size
    if over.size:
        worst = index_of(np.argmax(rel))
        assert explain is not None, (f"{label}: relative L2 vs oracle bf16 {rel.max():.3e} > {tol} "
                                     f"at row {worst}")
        assert rel.max() <= tol + 2.0 ** -7, (f"{label}: relative L2 vs oracle bf16 {rel.max():.3e} > "
                                              f"{tol + 2.0 ** -7} at row {worst}")
        assert over.size <= max(2, int(0.01 * rel.size)), (
            f"{label}: only {within:.4f} of the {rel.size} rows are within {tol}")
        for flat in over:
            index = index_of(flat)
            mine = got[index]
            flipped = None
            described = explain(index)
            candidates = described["rows"] if "rows" in described else ko.rounding_flip_rows(**described)
            for token, steps, bits in candidates:
                other = ko.bf16_to_f32(bits).reshape(mine.shape)
                if T.rel_l2(mine[None], other[None])[0] <= tol:
                    flipped = (token, steps)
                    break
            assert flipped, (f"{label}: row {index} is {rel.ravel()[flat]:.3e} from the oracle and no "
                             f"turned rounding of its heaviest tokens explains it")
    if explain is not None:
        ALLOWANCE_LOG.append((label, int(over.size), int(rel.size)))
    rel32 = T.rel_l2(got[rows_mask], want_f32[rows_mask])
    bound32 = np.full(rel32.shape, tol + 2e-3)
    bound32.ravel()[over] += 2.0 ** -7  # an explained row: one place of its heaviest weight more
    assert (rel32 <= bound32).all(), f"{label}: relative L2 vs oracle fp32 {rel32.max():.3e}"
    ulps = bf16_ulp_diff(out_bits[rows_mask], want_bits[rows_mask])
    return dict(rel_l2=float(rel.max()), rel_l2_mean=float(rel.mean()), rows_within_tol=within,
                rel_l2_fp32=float(rel32.max()), explained_rows=int(over.size),
                max_abs=float(np.abs(got[rows_mask] - want_f32[rows_mask]).max()),
                exact=float((ulps == 0).mean()), max_ulp=int(ulps.max()))


def lanes_explainer(fmt, kv_heads, group, head_dim, queries, tables, kv, committed, active, splits,
                    capacity, masks=None, one_row=False):
    """explain() for outputs indexed (lane, KV head, row, head in group) over verify-shaped
    queries [lane][KV head][row stride][group][D]; committed / active / splits per lane.
    one_row: outputs indexed (lane, KV head, head in group), row 0 (decode)."""
    def explain(index):
        if one_row:
            lane, head, g = index
            row = 0
        else:
            lane, head, row, g = index
        return dict(fmt=fmt, kv_heads=kv_heads, group=group, head_dim=head_dim,
                    tile_queries=queries[lane, head, :capacity].reshape(capacity * group, head_dim),
                    table=tables[lane], kv=kv, head=head, committed=int(committed[lane]),
                    active=int(active[lane] if np.ndim(active) else active), splits=int(splits[lane]),
                    capacity=capacity, fused_row=row * group + g,
                    masks=None if masks is None else masks[lane])
    return explain


def prefill_explainer(fmt, kv_heads, group, head_dim, queries, table, kv, committed, rows, splits):
    """explain() for outputs indexed (KV head, chunk row, head in group) of a chunked prefill
    over queries [KV head][chunk stride][group][D]: the row's 8-row tile."""
    def explain(index):
        head, row, g = index
        tile = row // 8
        tile_queries = np.zeros((8, group, head_dim), dtype=np.uint16)
        live = queries[head, 8 * tile:8 * tile + 8]
        tile_queries[:live.shape[0]] = live
        return dict(fmt=fmt, kv_heads=kv_heads, group=group, head_dim=head_dim,
                    tile_queries=tile_queries.reshape(8 * group, head_dim), table=table, kv=kv,
                    head=head, committed=committed + 8 * tile, active=min(8, rows - 8 * tile),
                    splits=splits, capacity=8, fused_row=(row % 8) * group + g)
    return explain


def oracle_tile(fmt, kv_heads, group, head_dim, tile_queries, table, kv, head, committed, active,
                splits, capacity, masks=None, score_scale=0.0):
    """The oracle's attention of one tile of one KV head (ko.attention_tile_rows)."""
    return ko.attention_tile_rows(fmt, kv_heads, group, head_dim, tile_queries, table, kv, head,
                                  committed, active, splits, capacity, masks, score_scale)
