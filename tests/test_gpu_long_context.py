"""Long histories on the matrix-core kernels: the reference's --long cases, 131 072 and 260 096
committed tokens (dev/tests/engine/paged_attention_plan_test.mm:999-1012), as a verify batch of
4 lanes x 8 rows, a one-row decode with the decode plan's hundreds of splits (the merge's four
ordered ranges) and a 257-row chunked prefill.  The oracle walks a quarter of a million tokens per
output row, so sampled rows are compared, each recomputed alone by the oracle; every call must
have run on the matrix-core kernels."""
import numpy as np
import pytest
import torch

from oracle import kvoracle as ko
from richengine_amd import kvx
import kvtestlib as T
import gpulib as Gp

pytestmark = pytest.mark.gpu
H, G, D = 4, 6, 256
QH = H * G
FMT = ko.INT4


def one_row(fmt, tile_queries, table, kv, head, committed, active, splits, capacity, fused_row):
    """One fused row of a tile by the oracle, the other rows skipped."""
    L = ko.lib()
    L.ko_attention_flips(fused_row, None, 0, 0.0, 1)   # no flips: that fused row alone
    try:
        bits, f32 = ko.attention_tile_rows(fmt, H, G, D, tile_queries, table, kv, head, committed,
                                           active, splits, capacity, only_row=fused_row)
    finally:
        L.ko_attention_flips(-1, None, 0, 0.0, 0)
    return bits[fused_row], f32[fused_row]


def check_row(got_bits, want_bits, want32, label, explain):
    got = got_bits.reshape(1, D)
    return Gp.check_attention(got, want_bits.reshape(1, D), want32.reshape(1, D),
                              np.ones(1, dtype=bool), 2e-3, label,
                              explain=lambda index: explain)


@pytest.mark.parametrize("history,FMT", [(131072, ko.INT4), (260096, ko.INT4), (131072, ko.INT8),
                                         (131072, ko.BF16)])
def test_long_history_verify_decode_and_prefill(history, FMT):
    rows = 257                                    # the prefill chunk; verify and decode sit inside it
    total = history + rows
    n_pages = (total + 31) // 32
    tw = Gp.Twin(FMT, H, D, 1, n_pages)
    pages = tw.pages(n_pages, history)
    th, td = tw.tables(pages)
    gen = torch.Generator(device="cuda").manual_seed(history)
    done = 0
    while done < total:                           # appended by the device, mirrored by its bytes
        n = min(2048, total - done)
        stride = (n + 31) // 32 * 32
        ck = torch.randn((H, stride, D), generator=gen, device="cuda").bfloat16()
        cv = torch.randn((H, D, stride), generator=gen, device="cuda").bfloat16()
        ck[:, :, [3, 77, 130, 255]] *= 20
        kvx.append(tw.dev, 0, ck.view(torch.int16), cv.view(torch.int16), [td],
                   [kvx.ChunkParams(done, n, stride, n_pages)], H * stride * D)
        done += n
    torch.cuda.synchronize()
    tw.download()
    kv = tw.host.layer(0)
    rng = np.random.default_rng(history)
    before = kvx.attend_paths()

    # ---- verify: 4 lanes x 8 rows over the same pages, the reference's split rule ----
    lanes = 4
    q = np.zeros((lanes, H, 32, G, D), dtype=np.uint16)
    q[:, :, :8] = ko.f32_to_bf16(rng.standard_normal((lanes, H, 8, G, D)).astype(np.float32)
                                 ).reshape(lanes, H, 8, G, D)
    splits = kvx.lib().kvx_verify_splits(history, 8)
    assert splits == 128
    dp = [kvx.VerifyParams(history, n_pages, kvx.KvLayer(), splits, splits, 8, 8, 0.0)] * lanes
    out = torch.full((lanes, H, 32, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
    kvx.attend_verify(tw.dev, 0, QH, Gp.dev(q), out, [td] * lanes, dp, None, 32, ws)
    torch.cuda.synchronize()
    got = Gp.host_u16(out)
    assert (got[:, :, 8:] == 0x5A5A).all()
    for lane, head, row, g in [(0, 0, 0, 0), (1, 3, 7, 5), (3, 2, 4, 1)]:
        args = dict(fmt=FMT, tile_queries=q[lane, head, :8].reshape(8 * G, D), table=th, kv=kv,
                    head=head, committed=history, active=8, splits=splits, capacity=8,
                    fused_row=row * G + g)
        want, want32 = one_row(**args)
        check_row(got[lane, head, row, g], want, want32, f"long verify fmt={FMT} {history} {lane, head, row, g}",
                  dict(kv_heads=H, group=G, head_dim=D, **args))

    # ---- decode: one row, the decode plan (hundreds of splits, merged in eight ranges) ----
    q1 = np.zeros((1, H, 1, G, D), dtype=np.uint16)
    q1[0, :, 0] = q[2, :, 0]
    splits = kvx.decode_plan([history], H, FMT)[0]
    assert splits > 32
    dp = [kvx.VerifyParams(history, n_pages, kvx.KvLayer(), splits, splits, 1, 1, 0.0)]
    out = torch.zeros((1, H, 1, G, D), dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
    kvx.attend_decode(tw.dev, 0, QH, Gp.dev(q1), out, [td], dp, 1, ws)
    torch.cuda.synchronize()
    got = Gp.host_u16(out)
    for head, g in [(0, 0), (2, 3), (3, 5)]:
        args = dict(fmt=FMT, tile_queries=q1[0, head, 0].reshape(G, D), table=th, kv=kv, head=head,
                    committed=history, active=1, splits=splits, capacity=1, fused_row=g)
        want, want32 = one_row(**args)
        check_row(got[0, head, 0, g], want, want32, f"long decode fmt={FMT} {history} {head, g} splits={splits}",
                  dict(kv_heads=H, group=G, head_dim=D, **args))

    # ---- chunked prefill: 257 rows, the split count sized for the GPU ----
    stride = 288
    qp = np.zeros((H, stride, G, D), dtype=np.uint16)
    qp[:, :rows] = ko.f32_to_bf16(rng.standard_normal((H, rows, G, D)).astype(np.float32)
                                  ).reshape(H, rows, G, D)
    splits = kvx.prefill_plan(history, rows, H, QH, FMT)
    assert splits > 1
    out = torch.full((H, stride, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.prefill_workspace_bytes(tw.dev, rows, QH, splits), dtype=torch.uint8,
                     device="cuda")
    kvx.attend_prefill(tw.dev, 0, QH, Gp.dev(qp), out, td,
                       kvx.PrefillParams(history, rows, stride, n_pages, kvx.KvLayer(), splits, 0.0), ws)
    torch.cuda.synchronize()
    got = Gp.host_u16(out)
    tile_end = (rows + 7) // 8 * 8
    assert not got[:, rows:tile_end].any() and (got[:, tile_end:] == 0x5A5A).all()
    for head, row, g in [(0, 0, 0), (1, 130, 4), (3, 256, 2), (2, 255, 5)]:
        tile = row // 8
        tile_queries = np.zeros((8, G, D), dtype=np.uint16)
        live = qp[head, 8 * tile:min(8 * tile + 8, rows)]
        tile_queries[:live.shape[0]] = live
        args = dict(fmt=FMT, tile_queries=tile_queries.reshape(8 * G, D), table=th, kv=kv, head=head,
                    committed=history + 8 * tile, active=min(8, rows - 8 * tile), splits=splits,
                    capacity=8, fused_row=(row % 8) * G + g)
        want, want32 = one_row(**args)
        check_row(got[head, row, g], want, want32, f"long prefill fmt={FMT} {history} {head, row, g}",
                  dict(kv_heads=H, group=G, head_dim=D, **args))

    after = kvx.attend_paths()
    assert after[1] == before[1] + 3 and after[0] == before[0], (before, after)
    tw.close()


def test_one_split_over_a_long_history():
    """The matrix-core kernels take a split of any length (their page entries come through the
    scalar unit as they go, not from a staged table): one split over 40 000 tokens (1251 pages),
    one-row decode."""
    history = 40000
    n_pages = (history + 1 + 31) // 32
    tw = Gp.Twin(FMT, H, D, 1, n_pages)
    pages = tw.pages(n_pages, 7)
    th, td = tw.tables(pages)
    gen = torch.Generator(device="cuda").manual_seed(7)
    done, total = 0, history + 1
    while done < total:
        n = min(2048, total - done)
        stride = (n + 31) // 32 * 32
        ck = torch.randn((H, stride, D), generator=gen, device="cuda").bfloat16()
        cv = torch.randn((H, D, stride), generator=gen, device="cuda").bfloat16()
        kvx.append(tw.dev, 0, ck.view(torch.int16), cv.view(torch.int16), [td],
                   [kvx.ChunkParams(done, n, stride, n_pages)], H * stride * D)
        done += n
    torch.cuda.synchronize()
    tw.download()
    rng = np.random.default_rng(7)
    q1 = ko.f32_to_bf16(rng.standard_normal((1, H, 1, G, D)).astype(np.float32)).reshape(1, H, 1, G, D)
    dp = [kvx.VerifyParams(history, n_pages, kvx.KvLayer(), 1, 1, 1, 1, 0.0)]
    out = torch.zeros((1, H, 1, G, D), dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
    before = kvx.attend_paths()
    kvx.attend_decode(tw.dev, 0, QH, Gp.dev(q1), out, [td], dp, 1, ws)
    torch.cuda.synchronize()
    after = kvx.attend_paths()
    assert after[1] == before[1] + 1 and after[0] == before[0]
    got = Gp.host_u16(out)
    for head, g in [(0, 0), (3, 5)]:
        want, want32 = one_row(FMT, q1[0, head, 0].reshape(G, D), th, tw.host.layer(0), head, history,
                               1, 1, 1, g)
        args = dict(fmt=FMT, tile_queries=q1[0, head, 0].reshape(G, D), table=th, kv=tw.host.layer(0),
                    head=head, committed=history, active=1, splits=1, capacity=1, fused_row=g)
        check_row(got[0, head, 0, g], want, want32, "one split over 1251 pages",
                  dict(kv_heads=H, group=G, head_dim=D, **args))
    tw.close()


def fill(tw, td, n_pages, total, seed):
    """History written by the device (bit-exactness of the append is other tests' business) and
    mirrored into the oracle's store by its bytes."""
    gen = torch.Generator(device="cuda").manual_seed(seed)
    done = 0
    while done < total:
        n = min(2048, total - done)
        stride = (n + 31) // 32 * 32
        ck = torch.randn((H, stride, D), generator=gen, device="cuda").clamp_(-6, 6).bfloat16()
        cv = torch.randn((H, D, stride), generator=gen, device="cuda").clamp_(-6, 6).bfloat16()
        kvx.append(tw.dev, 0, ck.view(torch.int16), cv.view(torch.int16), [td],
                   [kvx.ChunkParams(done, n, stride, n_pages)], H * stride * D)
        done += n
    torch.cuda.synchronize()
    tw.download()


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16, ko.FP8])
@pytest.mark.parametrize("history,rows", [(0, 2048), (4093, 1057), (16383, 257), (8064, 130), (6145, 2048)])
@pytest.mark.parametrize("planned", [False, True])
def test_reference_prefill_cases_on_sampled_rows(fmt, history, rows, planned):
    """The large cases of the reference's prefill list (dev/tests/engine/
    paged_attention_plan_test.mm:1018-1029; the small ones run whole in test_gpu_attention.py):
    full chunks, chunks that start one token before a page boundary and in the middle of a
    page, ragged last tiles.  Sampled rows, each recomputed alone by the oracle: the chunk's
    first and last rows, rows either side of a page boundary of the history, of a tile pair
    and of the last, partly filled tile.  With the reference's split rule and with the
    split count sized for the GPU."""
    total = history + rows
    n_pages = (total + 31) // 32
    tw = Gp.Twin(fmt, H, D, 1, n_pages)
    th, td = tw.tables(tw.pages(n_pages, history + rows))
    fill(tw, td, n_pages, total, history + 7 * rows)
    kv = tw.host.layer(0)
    rng = np.random.default_rng(history + rows)
    stride = (rows + 31) // 32 * 32
    qp = np.zeros((H, stride, G, D), dtype=np.uint16)
    qp[:, :rows] = ko.f32_to_bf16(rng.standard_normal((H, rows, G, D)).astype(np.float32)
                                  ).reshape(H, rows, G, D)
    splits = (kvx.prefill_plan(history, rows, H, QH, fmt) if planned
              else kvx.lib().kvx_prefill_splits(rows))
    out = torch.full((H, stride, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.prefill_workspace_bytes(tw.dev, rows, QH, splits), dtype=torch.uint8,
                     device="cuda")
    before = kvx.attend_paths()
    kvx.attend_prefill(tw.dev, 0, QH, Gp.dev(qp), out, td,
                       kvx.PrefillParams(history, rows, stride, n_pages, kvx.KvLayer(), splits, 0.0), ws)
    torch.cuda.synchronize()
    after = kvx.attend_paths()
    assert after[1] == before[1] + 1 and after[0] == before[0]      # the matrix-core kernels
    got = Gp.host_u16(out)
    tile_end = (rows + 7) // 8 * 8
    assert not got[:, rows:tile_end].any() and (got[:, tile_end:] == 0x5A5A).all()
    to_boundary = (32 - history % 32) % 32          # first chunk row that starts a page
    picks = {0, 7, 8, 15, 16, rows - 1, rows - 2, (rows - 1) // 8 * 8, rows // 2,
             to_boundary, max(to_boundary - 1, 0), to_boundary + 31, to_boundary + 32}
    picks = sorted(r for r in picks if 0 <= r < rows)
    tol = 1e-2 if fmt == ko.FP8 else 2e-3
    for i, row in enumerate(picks):
        head, g = (i * 5 + row) % H, (i * 7 + row) % G
        tile = row // 8
        tile_queries = np.zeros((8, G, D), dtype=np.uint16)
        live = qp[head, 8 * tile:min(8 * tile + 8, rows)]
        tile_queries[:live.shape[0]] = live
        args = dict(fmt=fmt, tile_queries=tile_queries.reshape(8 * G, D), table=th, kv=kv, head=head,
                    committed=history + 8 * tile, active=min(8, rows - 8 * tile), splits=splits,
                    capacity=8, fused_row=(row % 8) * G + g)
        want, want32 = one_row(**args)
        Gp.check_attention(got[head, row, g].reshape(1, D), want.reshape(1, D), want32.reshape(1, D),
                           np.ones(1, dtype=bool), tol,
                           f"reference prefill case fmt={fmt} {history}+{rows} splits={splits} "
                           f"{head, row, g}",
                           explain=lambda index: dict(kv_heads=H, group=G, head_dim=D, **args))
    tw.close()
