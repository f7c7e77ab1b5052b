"""QKV prepare fused with quantize-on-append (kv_prepare_append): per-head RMS norm,
partial rotary embedding, the layout change from packed projection rows to attention
queries, and keys / values quantized straight into their page slots (reference:
common/attention_qkv_prepare.h:12-83, common/rms_inverse.h:14-31, then the store
kernels).

CPU tests pin the oracle's restatement by mathematics (the reference holds no test
or vector of these kernels): float64 RMS norm and rotation, the layout against
numpy reshapes, and exact special cases (no norm and zero rotation copies the
bits; a quarter turn swaps the halves with one sign; the gate half of a query
head is never read).  Two choices of the restatement cannot be pinned against
the reference, whose simd_sum and rsqrt are Metal's: the order of the 32-lane sum
and the rounding of 1 / sqrt.

GPU tests hold kv_prepare_append to the oracle bit for bit: the queries, and every
byte of the pages against the oracle's prepare followed by the oracle's store.
"""
import ctypes as C

import numpy as np
import pytest

from oracle import kvoracle as ko
from richengine_amd import kvx


def bf16(x):
    x = np.asarray(x, dtype=np.float32)
    return ko.f32_to_bf16(x).reshape(x.shape)


def f32(bits):
    return ko.bf16_to_f32(bits).reshape(bits.shape)


def packed_rows(rng, tokens, heads, group, dim, gate, scale=1.0):
    width = heads * group * (2 if gate else 1) * dim + 2 * heads * dim
    return bf16(rng.standard_normal((tokens, width)) * scale)


def split_packed(packed, heads, group, dim, gate):
    """(query [T][QH][D], gate or None, keys [T][H][D], values [T][H][D]) by reshaping."""
    tokens, qh, qs = packed.shape[0], heads * group, (2 if gate else 1) * dim
    q = packed[:, :qh * qs].reshape(tokens, qh, qs)
    k = packed[:, qh * qs:qh * qs + heads * dim].reshape(tokens, heads, dim)
    v = packed[:, qh * qs + heads * dim:].reshape(tokens, heads, dim)
    return q[:, :, :dim], (q[:, :, dim:] if gate else None), k, v


def rope_tables(rng, tokens, pairs):
    angle = rng.uniform(-np.pi, np.pi, (tokens, pairs))
    return np.cos(angle).astype(np.float32), np.sin(angle).astype(np.float32)


def steps(a_bits, b_bits):
    def key(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, -(x & 0x7FFF), x & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


SHAPES = [(4, 6, 256, 32, True), (2, 8, 128, 64, False), (8, 4, 64, 32, False), (4, 1, 128, 32, True)]


# ------------------------------------------------------------- the oracle ----
@pytest.mark.parametrize("heads,group,dim,pairs,gate", SHAPES)
def test_no_norm_no_rotation_is_the_layout_change(heads, group, dim, pairs, gate):
    rng = np.random.default_rng(dim)
    tokens, stride = 11, 32
    packed = packed_rows(rng, tokens, heads, group, dim, gate)
    cos, sin = np.ones((tokens, pairs), np.float32), np.zeros((tokens, pairs), np.float32)
    q, k, v = ko.qkv_prepare(heads, group, dim, pairs, gate, 1e-6, tokens, stride, packed, None, None,
                             cos, sin)
    pq, _, pk, pv = split_packed(packed, heads, group, dim, gate)
    assert np.array_equal(q[:, :tokens], pq.reshape(tokens, heads, group, dim).transpose(1, 0, 2, 3))
    assert np.array_equal(k[:, :tokens], pk.transpose(1, 0, 2))
    assert np.array_equal(v[:, :, :tokens], pv.transpose(1, 2, 0))
    assert not q[:, tokens:].any() and not k[:, tokens:].any() and not v[:, :, tokens:].any()


@pytest.mark.parametrize("heads,group,dim,pairs,gate", SHAPES)
def test_quarter_turn_swaps_the_halves(heads, group, dim, pairs, gate):
    rng = np.random.default_rng(dim + 1)
    tokens = 5
    packed = packed_rows(rng, tokens, heads, group, dim, gate)
    cos, sin = np.zeros((tokens, pairs), np.float32), np.ones((tokens, pairs), np.float32)
    q, k, _ = ko.qkv_prepare(heads, group, dim, pairs, gate, 1e-6, tokens, 32, packed, None, None, cos,
                             sin)
    pq, _, pk, _ = split_packed(packed, heads, group, dim, gate)
    want = pq.reshape(tokens, heads, group, dim).transpose(1, 0, 2, 3).copy()
    first, second = want[..., :pairs].copy(), want[..., pairs:2 * pairs].copy()
    want[..., :pairs] = second ^ np.uint16(0x8000)  # first * 0 - second * 1
    want[..., pairs:2 * pairs] = first              # second * 0 + first * 1
    got = q[:, :tokens]
    # -0.0 and +0.0 aside (0 * x - y keeps y's sign flipped; zeros of the input are rare)
    assert np.array_equal(f32(got), f32(want))
    assert np.array_equal(f32(k[:, :tokens])[..., 2 * pairs:], f32(pk.transpose(1, 0, 2))[..., 2 * pairs:])


@pytest.mark.parametrize("heads,group,dim,pairs,gate", SHAPES)
@pytest.mark.parametrize("norm_dtype", ["bf16", "f32"])
def test_norm_and_rotation_against_float64(heads, group, dim, pairs, gate, norm_dtype):
    rng = np.random.default_rng(dim + 2)
    tokens, eps = 9, 1e-5
    packed = packed_rows(rng, tokens, heads, group, dim, gate, 3.0)
    wq, wk = bf16(1.0 + 0.3 * rng.standard_normal(dim)), bf16(1.0 + 0.3 * rng.standard_normal(dim))
    if norm_dtype == "f32":
        nq, nk = f32(wq), f32(wk)
    else:
        nq, nk = wq, wk
    ones, zeros = np.ones((tokens, pairs), np.float32), np.zeros((tokens, pairs), np.float32)
    # normalized rows are what an identity rotation lets through
    q_n, k_n, _ = ko.qkv_prepare(heads, group, dim, pairs, gate, eps, tokens, 32, packed, nq, nk, ones,
                                 zeros)
    pq, _, pk, _ = split_packed(packed, heads, group, dim, gate)
    for got, rows, weight in ((q_n[:, :tokens], pq.reshape(tokens, heads, group, dim).transpose(1, 0, 2, 3), wq),
                              (k_n[:, :tokens], pk.transpose(1, 0, 2), wk)):
        x = f32(rows).astype(np.float64)
        want = x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps) * f32(weight).astype(np.float64)
        d = steps(got, bf16(want))
        assert d.max() <= 1 and (d == 0).mean() > 0.99
    # the rotation of those normalized rows, against float64
    cos, sin = rope_tables(rng, tokens, pairs)
    q_r, k_r, _ = ko.qkv_prepare(heads, group, dim, pairs, gate, eps, tokens, 32, packed, nq, nk, cos, sin)
    for got, normal, per_row in ((q_r[:, :tokens], q_n[:, :tokens], lambda t: t[None, :, None, :]),
                                 (k_r[:, :tokens], k_n[:, :tokens], lambda t: t[None, :, :])):
        n = f32(normal).astype(np.float64)
        c, s = per_row(cos.astype(np.float64)), per_row(sin.astype(np.float64))
        want = n.copy()
        want[..., :pairs] = n[..., :pairs] * c - n[..., pairs:2 * pairs] * s
        want[..., pairs:2 * pairs] = n[..., pairs:2 * pairs] * c + n[..., :pairs] * s
        d = steps(got, bf16(want))
        assert d.max() <= 1 and (d == 0).mean() > 0.99
        assert np.array_equal(got[..., 2 * pairs:], normal[..., 2 * pairs:])


def test_gate_half_is_never_read_and_norm_types_agree():
    heads, group, dim, pairs = 4, 6, 256, 32
    rng = np.random.default_rng(3)
    tokens = 4
    packed = packed_rows(rng, tokens, heads, group, dim, True)
    w = bf16(1.0 + 0.2 * rng.standard_normal(dim))
    cos, sin = rope_tables(rng, tokens, pairs)
    a = ko.qkv_prepare(heads, group, dim, pairs, True, 1e-6, tokens, 32, packed, w, w, cos, sin)
    changed = packed.copy()
    view = changed[:, :heads * group * 2 * dim].reshape(tokens, heads * group, 2, dim)
    view[:, :, 1, :] = 0x7FC0  # NaN in every gate
    changed[:, :heads * group * 2 * dim] = view.reshape(tokens, -1)
    b = ko.qkv_prepare(heads, group, dim, pairs, True, 1e-6, tokens, 32, changed, w, w, cos, sin)
    c = ko.qkv_prepare(heads, group, dim, pairs, True, 1e-6, tokens, 32, packed, f32(w), f32(w), cos, sin)
    for x, y, z in zip(a, b, c):
        assert np.array_equal(x, y) and np.array_equal(x, z)


def test_library_exports_the_entry():
    assert hasattr(kvx.lib(), "kv_prepare_append")


# ---------------------------------------------------------------- the GPU ----
def fused_case(fmt, heads, group, dim, pairs, gate, norm, committed, tokens, rows, row_stride, seed,
               verify_max_rows=0):
    """Lanes with their own page tables in one pool; the oracle prepares and stores, the
    library does both in one call; queries and every page byte must agree."""
    import torch
    import gpulib as Gp
    rng = np.random.default_rng(seed)
    lanes, qh = len(committed), heads * group
    counts = [(c + t + 31) // 32 for c, t in zip(committed, tokens)]
    tw = Gp.Twin(fmt, heads, dim, 2, sum(counts))
    ids = tw.pages(sum(counts), seed)
    hts, dts, first = [], [], 0
    for n in counts:
        th, td = tw.tables(ids[first:first + n])
        first += n
        hts.append(th)
        dts.append(td)
    width = qh * (2 if gate else 1) * dim + 2 * heads * dim
    packed = bf16(rng.standard_normal((lanes, rows, width)) * 2.0)
    packed[0, 0, qh * (2 if gate else 1) * dim:qh * (2 if gate else 1) * dim + dim] = 0  # an all-zero key row
    angle = rng.uniform(-np.pi, np.pi, (lanes, rows, pairs))
    cos, sin = np.cos(angle).astype(np.float32), np.sin(angle).astype(np.float32)
    wq = wk = None
    if norm:
        wq, wk = bf16(1.0 + 0.3 * rng.standard_normal(dim)), bf16(1.0 + 0.3 * rng.standard_normal(dim))
        if norm == 2:
            wq, wk = f32(wq), f32(wk)
    eps = 1e-5 if dim == 64 else 1e-6
    stride = (max(tokens) + 31) // 32 * 32
    want_q = np.full((lanes, heads, row_stride, group, dim), 0x5A5A, dtype=np.uint16)
    for i in range(lanes):
        q, k, v = ko.qkv_prepare(heads, group, dim, pairs, gate, eps, tokens[i], stride, packed[i], wq,
                                 wk, cos[i], sin[i])
        want_q[i, :, :tokens[i]] = q[:, :tokens[i]]
        p = ko.ChunkParams(committed[i], tokens[i], stride, counts[i], tw.host.layer(1))
        assert ko.store_chunk(fmt, heads, dim, k, v, hts[i], p) == 1
    got_q = torch.full((lanes, heads, row_stride, group, dim), 0x5A5A, dtype=torch.int16, device="cuda")
    shape = kvx.QkvShape(qh, pairs, int(gate), norm, 0.0 if dim != 64 else 1e-5)
    dp = [kvx.ChunkParams(committed[i], tokens[i], 32 * ((tokens[i] + 31) // 32), counts[i])
          for i in range(lanes)]
    kvx.prepare_append(tw.dev, 1, shape, Gp.dev(packed), None if wq is None else Gp.dev(wq),
                       None if wk is None else Gp.dev(wk), Gp.dev(cos), Gp.dev(sin), got_q, row_stride,
                       dts, dp, rows, verify_max_rows)
    torch.cuda.synchronize()
    assert np.array_equal(Gp.host_u16(got_q), want_q), "prepared queries differ from the oracle"
    tw.assert_same_bytes()
    tw.close()


FORMATS = [ko.INT4, ko.INT8, ko.BF16, ko.FP8]


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", FORMATS)
def test_verify_rows_prepared_and_stored(fmt):
    fused_case(fmt, 4, 6, 256, 32, True, 1, [0, 1023, 1672, 31, 40, 27], [8, 8, 5, 8, 1, 6], 8, 32,
               seed=201, verify_max_rows=15)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", FORMATS)
def test_decode_rows_across_launches(fmt):
    rng = np.random.default_rng(9)
    committed = [int(c) for c in rng.integers(0, 3000, 40)]
    fused_case(fmt, 4, 6, 256, 32, True, 2, committed, [1] * 40, 1, 1, seed=203, verify_max_rows=15)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", FORMATS)
def test_prefill_chunk_prepared_and_stored(fmt):
    fused_case(fmt, 4, 6, 256, 32, True, 1, [77], [300], 300, 320, seed=205)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", FORMATS)
def test_long_chunks_of_unequal_lanes(fmt):
    """More than 32 768 (row, head) tasks in one call, lanes of very different length (so
    the kernel finds a task's lane by walking the lane records), a task count that is no
    multiple of a workgroup's four."""
    fused_case(fmt, 4, 6, 256, 32, True, 1, [77, 1000], [1230, 37], 1230, 1248, seed=211)


@pytest.mark.gpu
def test_long_chunk_of_a_narrower_head():
    fused_case(ko.INT4, 8, 4, 128, 64, False, 2, [5], [1030], 1030, 1056, seed=213)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [ko.INT4, ko.BF16])
@pytest.mark.parametrize("heads,group,dim,pairs,norm", [(2, 8, 128, 64, 0), (8, 4, 64, 32, 2)])
def test_other_head_dimensions(fmt, heads, group, dim, pairs, norm):
    fused_case(fmt, heads, group, dim, pairs, False, norm, [100, 31], [8, 3], 8, 32, seed=207,
               verify_max_rows=15)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [ko.INT4, ko.BF16])
@pytest.mark.parametrize("dim,pairs,gate", [(128, 32, True), (256, 32, False)])
def test_one_query_head_per_kv_head(fmt, dim, pairs, gate):
    """A group of one: every query head is its own KV head (the reciprocal that stands for
    the division by the group does not fit 32 bits there)."""
    fused_case(fmt, 4, 1, dim, pairs, gate, 1, [100, 31, 0], [8, 3, 5], 8, 32, seed=209,
               verify_max_rows=15)


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16])
@pytest.mark.parametrize("dim,pairs", [(256, 48), (128, 24), (64, 12)])
def test_shapes_of_the_workgroup_kernel(fmt, dim, pairs):
    """Rotary widths and head dimensions the one-wave-per-row kernel does not take (a pair's
    dimensions not a power-of-two number of lanes apart) run one workgroup per row; same
    bits."""
    fused_case(fmt, 2, 3, dim, pairs, True, 1, [100, 31, 0], [8, 3, 5], 8, 32, seed=209,
               verify_max_rows=15)


@pytest.mark.gpu
def test_prepare_rejects_bad_arguments():
    import torch
    import gpulib as Gp
    tw = Gp.Twin(ko.INT4, 4, 256, 2, 4)
    pages = tw.pages(2, 1)
    _, td = tw.tables(pages)
    before = [tw.dev.extent_read(e).copy() for e in range(tw.extents)]
    packed = torch.zeros((1, 8, 56 * 256), dtype=torch.int16, device="cuda")
    cos = torch.ones((1, 8, 32), dtype=torch.float32, device="cuda")
    q = torch.full((1, 4, 32, 6, 256), 0x5A5A, dtype=torch.int16, device="cuda")
    good = kvx.QkvShape(24, 32, 1, 0, 0.0)
    lane = [kvx.ChunkParams(10, 8, 32, 2)]
    cases = [
        (kvx.QkvShape(25, 32, 1, 0, 0.0), lane, 8),   # heads not a multiple
        (kvx.QkvShape(24, 129, 1, 0, 0.0), lane, 8),  # rotary pairs past the head
        (kvx.QkvShape(24, 32, 1, 1, 0.0), lane, 8),   # norm without weights
        (good, [kvx.ChunkParams(10, 9, 32, 2)], 8),    # more live rows than packed rows
        (good, [kvx.ChunkParams(60, 8, 32, 2)], 8),    # page table too short
    ]
    for shape, lanes, rows in cases:
        with pytest.raises(kvx.KvxError) as e:
            kvx.prepare_append(tw.dev, 1, shape, packed, None, None, cos, cos, q, 32, [td], lanes, rows)
        assert e.value.code == kvx.EINVAL
    torch.cuda.synchronize()
    assert (q == 0x5A5A).all()
    for e in range(tw.extents):
        assert np.array_equal(tw.dev.extent_read(e), before[e])
    tw.close()
