"""The merge's second output: the out-projection's operand written by the attention
merge itself, gated by the sigmoid of the packed projection rows or plainly
gathered (reference: decode/paged_attention.metal:266-330, 356-413, 466-530,
which must reproduce verify_attention_gate / verify_attention_gather,
decode/attention_qkv.metal:121-164, bit for bit).

CPU tests pin the oracle's restatement by mathematics, since the reference's only
check of these kernels is a Metal fused-against-unfused comparison: the sigmoid
against identities and float64, the index map against an independent
transpose / reshape statement in numpy.  GPU tests then compare the fused entry
with the oracle applied to the rows kv_attend_verify stages:
  - the staged rows are the same bits with and without the second output;
  - gathered hidden rows are bit-exact;
  - gated rows differ by at most one bf16 step (the exp2 of the GPU and of the
    host libm may differ in the last bit of the float), and nearly all are exact.
"""
import ctypes as C

import numpy as np
import pytest

from oracle import kvoracle as ko
from richengine_amd import kvx


def rand_bf16(rng, shape, scale=1.0):
    return ko.f32_to_bf16((rng.standard_normal(shape) * scale).astype(np.float32)).reshape(shape)


def as_f64(bits):
    return ko.bf16_to_f32(bits).reshape(bits.shape).astype(np.float64)


# ------------------------------------------------------------- the oracle ----
def test_sigmoid_identities_and_float64():
    L = ko.lib()
    assert L.ko_sigmoid(0.0) == 0.5
    assert L.ko_sigmoid(200.0) == 1.0 and L.ko_sigmoid(-200.0) == 0.0
    xs = np.concatenate([np.linspace(-30, 30, 601), [1e-3, -1e-3, 17.5, -17.5]]).astype(np.float32)
    got = np.array([L.ko_sigmoid(float(x)) for x in xs], dtype=np.float32)
    want = 1.0 / (1.0 + np.exp(-xs.astype(np.float64)))
    # the product x * log2(e) is rounded to a float, which moves 2^(...) by up to
    # |x| * 2^-24 * ln 2 relative; the exp2, the sum and the quotient add an ulp each
    assert np.all(np.abs(got - want) <= want * (np.abs(xs) * 6e-8 + 3e-7))
    mirrored = np.array([L.ko_sigmoid(float(-x)) for x in xs], dtype=np.float32)
    assert np.all(np.abs(got.astype(np.float64) + mirrored - 1.0) < 3e-7)
    assert np.all(np.diff(got[:601]) >= 0)  # monotone


@pytest.mark.parametrize("kv_heads,group,dim,rows,stride", [(4, 6, 256, 8, 32), (2, 8, 128, 16, 32),
                                                          (8, 5, 64, 1, 1), (3, 2, 64, 5, 7)])
def test_hidden_index_map_is_a_transpose(kv_heads, group, dim, rows, stride):
    """Gather: hidden[lane][row][kv head * group + g][d] = attention[lane][kv head][row][g][d],
    stated here as a transpose of distinct values."""
    lanes = 3
    attention = (np.arange(lanes * kv_heads * stride * group * dim, dtype=np.uint32) % 65521).astype(
        np.uint16).reshape(lanes, kv_heads, stride, group, dim)
    # keep every pattern a finite bf16 (the gather round-trips through float)
    attention &= np.uint16(0x7F7F)
    hidden = ko.attention_hidden(kv_heads, group, dim, rows, attention)
    want = attention[:, :, :rows].transpose(0, 2, 1, 3, 4).reshape(lanes, rows, kv_heads * group, dim)
    assert np.array_equal(hidden, want)


@pytest.mark.parametrize("kv_heads,group,dim,rows", [(4, 6, 256, 8), (2, 8, 256, 16), (4, 4, 256, 1)])
def test_gate_reads_the_gate_half_of_each_query_head(kv_heads, group, dim, rows):
    rng = np.random.default_rng(kv_heads * 100 + rows)
    lanes, qh = 2, kv_heads * group
    attention = rand_bf16(rng, (lanes, kv_heads, 32, group, dim))
    packed = rand_bf16(rng, (lanes, rows, (2 * qh + 2 * kv_heads) * dim), 3.0)
    hidden = ko.attention_hidden(kv_heads, group, dim, rows, attention, packed)
    # independent statement: split the packed row into its parts by reshaping
    gates = packed[:, :, :2 * qh * dim].reshape(lanes, rows, qh, 2, dim)[:, :, :, 1, :]
    values = attention[:, :, :rows].transpose(0, 2, 1, 3, 4).reshape(lanes, rows, qh, dim)
    want = as_f64(values) / (1.0 + np.exp(-as_f64(gates)))
    got = as_f64(hidden)
    assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -8 + 1e-30)  # one bf16 rounding
    # a zero gate halves the value exactly, whatever the query half holds
    packed0 = packed.copy().reshape(lanes, rows, -1)
    view = packed0[:, :, :2 * qh * dim].reshape(lanes, rows, qh, 2, dim)
    view[:, :, :, 1, :] = 0
    packed0[:, :, :2 * qh * dim] = view.reshape(lanes, rows, -1)
    halved = ko.attention_hidden(kv_heads, group, dim, rows, attention, packed0)
    assert np.array_equal(as_f64(halved), as_f64(values) * 0.5)


def test_library_exports_the_entry():
    assert hasattr(kvx.lib(), "kv_attend_verify_hidden")
    assert hasattr(kvx.lib(), "kv_append_attend_decode_hidden")


# ---------------------------------------------------------------- the GPU ----
H, G, D = 4, 6, 256
QH = H * G


def fused_against_staged(tw, fmt, heads, group, dim, dts, dp, masks, capacity, row_stride, seed,
                         expect_matrix):
    """Runs kv_attend_verify and both modes of kv_attend_verify_hidden on the same lanes and
    checks the second output against the oracle applied to the staged rows."""
    import torch
    import gpulib as Gp
    import test_gpu_attention as A
    lanes, qh = len(dp), heads * group
    rng = np.random.default_rng(seed)
    q = np.zeros((lanes, heads, row_stride, group, dim), dtype=np.uint16)
    q[:, :, :capacity] = A.queries((lanes, heads, capacity, group, dim), seed)
    packed = rand_bf16(rng, (lanes, capacity, (2 * qh + 2 * heads) * dim), 2.0)
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, qh), dtype=torch.uint8, device="cuda")
    shape = (lanes, heads, row_stride, group, dim)
    dmasks = Gp.dev(masks) if masks is not None else None
    staged = torch.full(shape, 0x5A5A, dtype=torch.int16, device="cuda")
    before = kvx.attend_paths()
    kvx.attend_verify(tw.dev, 1, qh, Gp.dev(q), staged, dts, dp, dmasks, row_stride, ws)
    staged_too = torch.full(shape, 0x5A5A, dtype=torch.int16, device="cuda")
    gated = torch.full((lanes, capacity, qh, dim), 0x3C3C, dtype=torch.int16, device="cuda")
    kvx.attend_verify_hidden(tw.dev, 1, qh, Gp.dev(q), staged_too, dts, dp, dmasks, row_stride, ws,
                             Gp.dev(packed), gated)
    gathered = torch.full((lanes, capacity, qh, dim), 0x3C3C, dtype=torch.int16, device="cuda")
    kvx.attend_verify_hidden(tw.dev, 1, qh, Gp.dev(q), None, dts, dp, dmasks, row_stride, ws, None,
                             gathered)
    torch.cuda.synchronize()
    after = kvx.attend_paths()
    generic, matrix = after[0] - before[0], after[1] - before[1]
    assert (matrix == 3 and generic == 0) if expect_matrix else (generic == 3 and matrix == 0)
    assert torch.equal(staged, staged_too), "staged rows changed with the second output"
    rows = Gp.host_u16(staged)
    assert np.array_equal(Gp.host_u16(gathered), ko.attention_hidden(heads, group, dim, capacity, rows))
    want = ko.attention_hidden(heads, group, dim, capacity, rows, packed)
    got = Gp.host_u16(gated)
    steps = Gp.bf16_ulp_diff(got, want)
    assert steps.max() <= 1, f"gated rows are {steps.max()} bf16 steps from the oracle"
    assert (steps == 0).mean() > 0.995
    for lane, p in enumerate(dp):  # rows past the live ones are zeros in both outputs
        assert not got[lane, p.active_rows:].any()
        assert not Gp.host_u16(gathered)[lane, p.active_rows:].any()
        assert got[lane, :p.active_rows].any()
    return got


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16, ko.FP8])
def test_chain_verify_hidden_rows(fmt):
    import test_gpu_attention as A
    committed = [0, 1023, 1672, 31, 40]  # one page (a single split) up to 53 pages
    tw, counts, hts, dts = A.shared_pool_lanes(fmt, committed, 8, seed=141)
    active = [8, 8, 5, 8, 1]
    splits = [kvx.lib().kvx_verify_splits(c, 8) for c in committed]
    splits[4] = 1
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], 128, active[i], 8, 0.0)
          for i in range(len(committed))]
    fused_against_staged(tw, fmt, H, G, D, dts, dp, None, 8, 32, 11, True)
    tw.close()


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [ko.INT4, ko.BF16])
def test_tree_verify_hidden_rows(fmt):
    import test_gpu_attention as A
    committed, nodes = [260, 31, 4000], 15
    tw, counts, hts, dts = A.shared_pool_lanes(fmt, committed, nodes, seed=171)
    rng = np.random.default_rng(3)
    masks = np.zeros((len(committed), 16), dtype=np.uint32)
    for lane in range(len(committed)):
        parents = [-1] + [int(rng.integers(max(0, i - 3), i)) for i in range(1, nodes)]
        masks[lane, :nodes] = A.tree_masks(parents)
    splits = [kvx.lib().kvx_verify_splits(c, nodes) for c in committed]
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], 128, nodes, 16, 0.0)
          for i in range(len(committed))]
    fused_against_staged(tw, fmt, H, G, D, dts, dp, masks, 16, 32, 13, True)
    tw.close()


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8])
def test_decode_hidden_rows_across_launches(fmt):
    """One-row lanes, more than one launch holds (32): the second launch's rows must land
    after the first's."""
    import test_gpu_attention as A
    rng = np.random.default_rng(5)
    committed = [int(c) for c in rng.integers(0, 2500, 40)]
    committed[7], committed[33] = 0, 31
    tw, counts, hts, dts = A.shared_pool_lanes(fmt, committed, 1, seed=191)
    splits = [0] * len(committed)
    plan = (C.c_uint32 * len(committed))()
    kvx.check(kvx.lib().kvx_decode_plan((C.c_uint32 * len(committed))(*committed), len(committed), H,
                                        fmt, plan))
    splits = list(plan)
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], splits[i], 1, 1, 0.0)
          for i in range(len(committed))]
    fused_against_staged(tw, fmt, H, G, D, dts, dp, None, 1, 1, 17, True)
    tw.close()


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16])
def test_append_attend_decode_hidden_is_the_two_calls(fmt):
    """kv_append_attend_decode_hidden: the page bytes of kv_append, and the staged and hidden rows
    of kv_attend_verify_hidden over them, bit for bit, gated and gathered, with and without the
    staged rows; int4 pages take the kernel that stores the token itself, 40 lanes two launches."""
    import torch
    import gpulib as Gp
    import kvtestlib as T
    import test_gpu_attention as A
    rng = np.random.default_rng(77)
    committed = [0, 31, 32, 700, 4095, 1000, 63, 2047] + [int(c) for c in rng.integers(0, 1500, 32)]
    lanes = len(committed)
    tw, counts, hts, dts = A.shared_pool_lanes(fmt, committed, 1, seed=78)
    k = rng.standard_normal((lanes, H, 1, D)).astype(np.float32)
    v = rng.standard_normal((lanes, H, 1, D)).astype(np.float32)
    ck = np.zeros((lanes, H, 32, D), dtype=np.uint16)
    cv = np.zeros((lanes, H, D, 32), dtype=np.uint16)
    for lane in range(lanes):
        ck[lane], cv[lane] = T.chunk_buffers(k[lane], v[lane], 32)
    q = A.queries((lanes, H, 1, G, D), 79)
    packed = rand_bf16(rng, (lanes, 1, (2 * QH + 2 * H) * D), 2.0)
    plan = (C.c_uint32 * lanes)()
    kvx.check(kvx.lib().kvx_decode_plan((C.c_uint32 * lanes)(*committed), lanes, H, fmt, plan))
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), plan[i], plan[i], 1, 1, 0.0)
          for i in range(lanes)]
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
    before = [tw.dev.extent_read(e).copy() for e in range(tw.extents)]
    dq, dk, dv, dpacked = Gp.dev(q), Gp.dev(ck), Gp.dev(cv), Gp.dev(packed)

    def fresh(shape, fill):
        return torch.full(shape, fill, dtype=torch.int16, device="cuda")

    # the two calls, gated and gathered
    kvx.append(tw.dev, 1, dk, dv, dts, [kvx.ChunkParams(committed[i], 1, 32, counts[i]) for i in range(lanes)],
               H * 32 * D)
    want_rows, want_gated = fresh((lanes, H, 1, G, D), 0x5A5A), fresh((lanes, 1, QH, D), 0x3C3C)
    kvx.attend_verify_hidden(tw.dev, 1, QH, dq, want_rows, dts, dp, None, 1, ws, dpacked, want_gated)
    want_gathered = fresh((lanes, 1, QH, D), 0x3C3C)
    kvx.attend_verify_hidden(tw.dev, 1, QH, dq, None, dts, dp, None, 1, ws, None, want_gathered)
    torch.cuda.synchronize()
    after_two = [tw.dev.extent_read(e).copy() for e in range(tw.extents)]
    assert want_gated.any() and want_gathered.any()
    for gated in (True, False):
        for e in range(tw.extents):
            tw.dev.extent_write(e, before[e])
        ws.fill_(0xA5)
        rows, hidden = fresh((lanes, H, 1, G, D), 0x5A5A), fresh((lanes, 1, QH, D), 0x3C3C)
        paths = kvx.attend_paths()
        kvx.append_attend_decode_hidden(tw.dev, 1, dk, dv, H * 32 * D, 32, QH, dq, rows if gated else None,
                                        dts, dp, 1, ws, dpacked if gated else None, hidden)
        torch.cuda.synchronize()
        assert kvx.attend_paths()[1] > paths[1] and kvx.attend_paths()[0] == paths[0]
        assert torch.equal(hidden, want_gated if gated else want_gathered)
        if gated:
            assert torch.equal(rows, want_rows)
        for e in range(tw.extents):
            assert np.array_equal(tw.dev.extent_read(e), after_two[e])
    with pytest.raises(kvx.KvxError):
        kvx.append_attend_decode_hidden(tw.dev, 1, dk, dv, H * 32 * D, 32, QH, dq, None, dts, dp, 1, ws,
                                        dpacked, None)
    tw.close()


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [ko.INT4, ko.BF16])
@pytest.mark.parametrize("heads,group,dim", [(2, 8, 128), (8, 4, 64)])
def test_other_head_dimensions_hidden_rows(fmt, heads, group, dim):
    """The no-gate targets of the reference (head dimensions 128 and 64) run on the
    format-generic kernels; both modes are covered there too."""
    import gpulib as Gp
    import test_gpu_attention as A
    committed, rows = 300, 8
    tw = Gp.Twin(fmt, heads, dim, 2, (committed + rows + 31) // 32)
    pages, th, td = A.fill(tw, committed + rows, seed=dim + heads)
    splits = kvx.lib().kvx_verify_splits(committed, rows)
    dp = [kvx.VerifyParams(committed, len(pages), kvx.KvLayer(), splits, 128, 7, 8, 0.0)]
    fused_against_staged(tw, fmt, heads, group, dim, [td], dp, None, 8, 32, 19, False)
    tw.close()


@pytest.mark.gpu
def test_hidden_entry_rejects_bad_arguments():
    import torch
    import test_gpu_attention as A
    tw, counts, hts, dts = A.shared_pool_lanes(ko.INT4, [100], 8, seed=7)
    dp = [kvx.VerifyParams(100, counts[0], kvx.KvLayer(), 32, 128, 8, 8, 0.0)]
    q = torch.zeros((1, H, 32, G, D), dtype=torch.int16, device="cuda")
    out = torch.full((1, H, 32, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    hidden = torch.full((1, 8, QH, D), 0x3C3C, dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
    for args in ((out, None, None), (out, None, out), (q, None, hidden)):
        with pytest.raises(kvx.KvxError) as e:
            kvx.attend_verify_hidden(tw.dev, 1, QH, q, args[0], dts, dp, None, 32, ws, args[1], args[2])
        assert e.value.code == kvx.EINVAL
    torch.cuda.synchronize()
    assert (out == 0x5A5A).all() and (hidden == 0x3C3C).all()  # nothing was enqueued
    tw.close()
