"""The merge kernels alone (kv_attend_merge), fed the reference's synthetic partial rows and
statistics -- maxima up to 2000 apart, so that weights underflow, next to fractional ones,
ragged sums, inactive rows -- and compared with the fp64 merge at the reference's bound
|got - want| <= 0.004 |want| + 2e-6 (dev/tests/engine/q8_flash_attention_metal_test.mm:648-725).
One to 512 splits: up to 32 are summed in split order by one wave, more in eight ordered ranges.
The same rows through kv_attend_split + kv_attend_merge must give kv_attend_verify's bits."""
import numpy as np
import pytest
import torch

from oracle import kvoracle as ko
from richengine_amd import kvx
import gpulib as Gp
import test_gpu_attention as A

pytestmark = pytest.mark.gpu
D = 256


def pattern(heads, splits, m, group, active):
    h_idx, s_idx, r_idx = np.meshgrid(np.arange(heads), np.arange(splits), np.arange(m), indexing="ij")
    act = (r_idx // group) < active
    spacing = np.where(r_idx % 2 == 1, 0.25, 500.0)
    mx = np.where(act, ((s_idx % 5) - 2) * spacing, -np.inf).astype(np.float32)
    sm = np.where(act, 1.0 + (s_idx % 7), 0.0).astype(np.float32)
    d_idx = np.arange(D)
    part = (((s_idx[..., None] * 71 + d_idx * 37 + r_idx[..., None] * 13) % 257) - 128) * 0.125
    return part.astype(np.float32), np.stack([mx, sm], axis=-1).astype(np.float32)


@pytest.mark.parametrize("heads,group", [(4, 6), (2, 8), (4, 4)])
@pytest.mark.parametrize("splits,capacity,active", [(1, 8, 8), (5, 8, 8), (32, 8, 8), (128, 8, 8),
                                                    (7, 8, 3), (33, 8, 8), (512, 1, 1), (77, 1, 1),
                                                    (128, 16, 15)])
def test_merge_alone_against_the_fp64_merge(heads, group, splits, capacity, active):
    m = capacity * group
    part, stats = pattern(heads, splits, m, group, active)
    storage = kvx.Storage(1, heads, D, kvx.INT4, 4, 4)          # the merge reads no page
    # committed so that every split owns a page: pages = splits
    committed = splits * 32 - active
    lane = kvx.VerifyParams(committed, splits, kvx.KvLayer(), splits, splits, active, capacity, 0.0)
    rows = heads * splits * m
    statistics_at = (rows * D * 4 + 255) // 256 * 256
    ws = torch.zeros(statistics_at + rows * 8, dtype=torch.uint8, device="cuda")
    ws[:rows * D * 4] = torch.from_numpy(part.reshape(-1).view(np.uint8)).cuda()
    ws[statistics_at:] = torch.from_numpy(stats.reshape(-1).view(np.uint8)).cuda()
    assert ws.numel() <= kvx.attend_workspace_bytes(storage, [lane], heads * group) + 256
    out = torch.full((1, heads, 32, group, D), 0x5A5A, dtype=torch.int16, device="cuda")
    before = kvx.attend_paths()
    kvx.attend_merge(storage, heads * group, out, [lane], 32, ws)
    torch.cuda.synchronize()
    assert kvx.attend_paths()[1] == before[1] + 1               # the matrix-core merge kernel
    got = ko.bf16_to_f32(Gp.host_u16(out)).reshape(heads, 32, group, D)[:, :capacity].reshape(heads, m, D)
    raw = Gp.host_u16(out).reshape(heads, 32, group, D)
    assert (raw[:, capacity:] == 0x5A5A).all()                   # nothing past the lane's rows
    mx, sm = stats[..., 0].astype(np.float64), stats[..., 1].astype(np.float64)
    for head in range(heads):
        for row in range(m):
            if row // group >= active:
                assert not got[head, row].any()
                continue
            w = np.exp(mx[head, :, row] - mx[head, :, row].max())
            want = (w[:, None] * part[head, :, row].astype(np.float64)).sum(0) / (w * sm[head, :, row]).sum()
            assert np.all(np.abs(got[head, row] - want) <= np.abs(want) * 0.004 + 2e-6), (head, row)
    # the oracle's merge (split order, fp32) on the same rows: bf16 results a place apart at most
    L = ko.lib()
    for head in (0, heads - 1):
        for row in range(0, active * group, 5):
            bits = np.zeros(D, dtype=np.uint16)
            L.ko_attention_reduce_row(group, D, capacity, ko.ptr(np.ascontiguousarray(part[head])),
                                      ko.ptr(np.ascontiguousarray(stats[head])), committed, active,
                                      splits, 0, row, ko.ptr(bits), None)
            mine = raw[head, row // group, row % group]
            assert Gp.bf16_ulp_diff(mine, bits).max() <= (0 if splits <= 32 else 1), (head, row)
    storage.close()


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16, ko.FP8])
def test_split_then_merge_is_the_verify_call(fmt):
    H, G = A.H, A.G
    committed = [0, 1023, 1672, 31, 1980]
    tw, counts, hts, dts = A.shared_pool_lanes(fmt, committed, 8, seed=141)
    lanes = len(committed)
    q = np.zeros((lanes, H, 32, G, D), dtype=np.uint16)
    q[:, :, :8] = A.queries((lanes, H, 8, G, D), 15)
    splits = [1, 32, 40, 1, 3]
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], 0, 8, 8, 0.0)
          for i in range(lanes)]
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, H * G), dtype=torch.uint8, device="cuda")
    one = torch.full((lanes, H, 32, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    kvx.attend_verify(tw.dev, 1, H * G, Gp.dev(q), one, dts, dp, None, 32, ws)
    two = torch.full_like(one, 0x5A5A)
    ws.fill_(0xA5)
    kvx.attend_split(tw.dev, 1, H * G, Gp.dev(q), dts, dp, None, 32, ws)
    kvx.attend_merge(tw.dev, H * G, two, dp, 32, ws)
    torch.cuda.synchronize()
    assert torch.equal(one, two)
    tw.close()


def test_decode_call_is_split_then_merge():
    """kv_attend_decode over a mixed batch gives the bits of kv_attend_split followed by
    kv_attend_merge: lanes of one split (written by the split call), of two to 32, more than 32
    lanes (several launches), repeated calls over a dirty workspace, and three streams at
    once."""
    H, G = A.H, A.G
    rng = np.random.default_rng(7)
    committed = [int(c) for c in rng.integers(1, 3000, 40)] + [0, 31, 32, 1023, 1024, 2047]
    tw, counts, hts, dts = A.shared_pool_lanes(ko.INT4, committed, 1, seed=143)
    lanes = len(committed)
    q = A.queries((lanes, H, 1, G, D), 17)
    splits = [min(max(1, counts[i] // (1 + i % 5)), 40) for i in range(lanes)]
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], splits[i], 1, 1, 0.0)
          for i in range(lanes)]
    ws_bytes = kvx.attend_workspace_bytes(tw.dev, dp, H * G)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    want = torch.full((lanes, H, 1, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    kvx.attend_split(tw.dev, 1, H * G, Gp.dev(q), dts, dp, None, 1, ws)
    kvx.attend_merge(tw.dev, H * G, want, dp, 1, ws)
    torch.cuda.synchronize()
    for _ in range(3):
        ws.fill_(0xA5)
        got = torch.full_like(want, 0x5A5A)
        kvx.attend_decode(tw.dev, 1, H * G, Gp.dev(q), got, dts, dp, 1, ws)
        torch.cuda.synchronize()
        assert torch.equal(got, want)
    streams = [torch.cuda.Stream() for _ in range(3)]
    spaces = [torch.empty(ws_bytes, dtype=torch.uint8, device="cuda") for _ in streams]
    outs = [torch.full_like(want, 0x5A5A) for _ in streams]
    qd = Gp.dev(q)
    torch.cuda.synchronize()
    for turn in range(4):
        for s, space, out in zip(streams, spaces, outs):
            kvx.attend_decode(tw.dev, 1, H * G, qd, out, dts, dp, 1, space, stream=s.cuda_stream)
    torch.cuda.synchronize()
    for out in outs:
        assert torch.equal(out, want)
    tw.close()


@pytest.mark.gpu
def test_calibration_stream_runs_and_rejects_what_it_does_not_cover():
    """kvx_calibrate_stream: the int4 decode kernel's loads alone.  It has no output to compare;
    the test is that it runs to completion over a shuffled table with every grouping of heads,
    leaves its sink word alone, and refuses other formats and head groupings."""
    L = kvx.lib()
    twin = Gp.Twin(kvx.INT4, 4, 256, 2, 40)
    try:
        pages = twin.pages(37, seed=5)
        _, table = twin.tables(pages)
        sink = torch.zeros(1, dtype=torch.int32, device="cuda")
        for heads in (1, 2, 4):
            for per in (1, 5, 64):
                assert L.kvx_calibrate_stream(twin.dev.h, 1, table.data_ptr(), len(pages), per, heads,
                                              sink.data_ptr(), None) == 0
        # the forms that are not the kernel's shape: 16-byte loads of whole KiB with 1, 2 or 4
        # pages ahead at 1 to 8 waves per SIMD, and the linear read of as many bytes
        for depth in (1, 2, 4):
            for waves in (1, 2, 4, 8):
                assert L.kvx_calibrate_stream_form(twin.dev.h, 1, table.data_ptr(), len(pages), 5,
                                                   1, depth, waves, sink.data_ptr(), None) == 0
        assert L.kvx_calibrate_stream_form(twin.dev.h, 1, None, 4, 2, 2, 1, 8, sink.data_ptr(), None) == 0
        torch.cuda.synchronize()
        assert int(sink.item()) == 0
        for form, depth, waves, count in ((1, 3, 2, 4), (1, 2, 3, 4), (7, 1, 2, 4), (2, 1, 8, 1 << 20)):
            assert L.kvx_calibrate_stream_form(twin.dev.h, 1, table.data_ptr(), count, 2, form, depth,
                                               waves, sink.data_ptr(), None) == -1
        assert L.kvx_calibrate_stream(twin.dev.h, 1, table.data_ptr(), len(pages), 4, 3,
                                      sink.data_ptr(), None) == -1
        assert L.kvx_calibrate_stream(twin.dev.h, 2, table.data_ptr(), len(pages), 4, 1,
                                      sink.data_ptr(), None) != 0
    finally:
        twin.close()
    other = Gp.Twin(kvx.BF16, 4, 256, 1, 8)
    try:
        _, table = other.tables(other.pages(4, seed=1))
        sink = torch.zeros(1, dtype=torch.int32, device="cuda")
        assert L.kvx_calibrate_stream(other.dev.h, 0, table.data_ptr(), 4, 2, 1, sink.data_ptr(),
                                      None) == -1
    finally:
        other.close()
