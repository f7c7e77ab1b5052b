"""GPU parity of paged attention (decode, chain / tree verify, chunked prefill)
against the oracle on the same seeded inputs, through the C ABI.

Bar: per output row, ||gpu - oracle||2 / ||oracle||2 <= 2e-3 for int4 / int8 /
bf16 pages and <= 1e-2 for fp8 pages, on the bf16 outputs (gpulib.check_attention
says why the oracle's fp32 value gets 2e-3 more).
"""
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
FORMATS = [ko.INT4, ko.INT8, ko.BF16, ko.FP8]
# every format runs on the matrix-core kernels at head dimension 256 and a GQA
# group of at most 16; other shapes run on the format-generic kernels
MATRIX = tuple(FORMATS)


@pytest.fixture(autouse=True)
def which_kernels_ran(request):
    """Pages of head dimension 256 with a group of at most 16 query heads must run
    on the matrix-core kernels and the other shapes (tests with a `dim`
    parameter) on the format-generic ones: a test that passed through the other
    path would not have tested what it names."""
    before = kvx.attend_paths()
    yield
    after = kvx.attend_paths()
    fmt = request.node.callspec.params.get("fmt") if hasattr(request.node, "callspec") else None
    if fmt is None:
        return
    generic, matrix = after[0] - before[0], after[1] - before[1]
    if "dim" not in request.node.callspec.params:
        assert matrix > 0 and generic == 0, (generic, matrix)
    else:
        assert generic > 0 and matrix == 0, (generic, matrix)


def tol(fmt):
    return 1e-2 if fmt == ko.FP8 else 2e-3


def fill(tw, total, seed, layer=1, scale=1.0, pages=None):
    """Appends `total` tokens on the device (the path under test) and mirrors
    them into the oracle store by copying the device bytes back."""
    n_pages = (total + 31) // 32
    if pages is None:
        pages = tw.pages(n_pages, seed)
    assert len(pages) == n_pages
    th, td = tw.tables(pages)
    rng = np.random.default_rng(seed)
    done = 0
    while done < total:
        n = min(2048, total - done)
        k = (rng.standard_normal((tw.H, n, tw.D)) * scale).astype(np.float32)
        v = (rng.standard_normal((tw.H, n, tw.D)) * scale).astype(np.float32)
        k[:, :, [c for c in (3, 77, 130, 255) if c < tw.D]] *= 20
        stride = (n + 31) // 32 * 32
        ck, cv = T.chunk_buffers(k, v, stride)
        kvx.append(tw.dev, layer, Gp.dev(ck), Gp.dev(cv), [td],
                   [kvx.ChunkParams(done, n, stride, n_pages)], tw.H * stride * tw.D)
        p = ko.ChunkParams(done, n, stride, n_pages, tw.host.layer(layer))
        assert ko.store_chunk(tw.fmt, tw.H, tw.D, ck, cv, th, p) == 1
        done += n
    torch.cuda.synchronize()
    return pages, th, td


def queries(shape_rows, seed):
    """bf16 queries for [..., rows, G, D]-shaped tiles."""
    rng = np.random.default_rng(seed + 999)
    return ko.f32_to_bf16(rng.standard_normal(shape_rows).astype(np.float32)).reshape(shape_rows)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("committed,rows", [(0, 1), (33, 7), (255, 17), (1023, 8), (100, 77),
                                            (2000, 130), (1500, -136), (1508, -136)])
def test_prefill_matches_oracle(fmt, committed, rows):
    # rows < 0: that many rows with kvx_prefill_plan's split count in place of the
    # reference rule's (which gives 136 and 264 rows a single split); after 1500 tokens the
    # tiles stay paired under several splits, after 1508 they run one by one.  1500
    # is 4 tokens before a page boundary, so the rows of the first pair of tiles see
    # different parts of two pages
    prefill_case(fmt, committed, rows)


def test_int4_prefill_pairs_tiles_under_several_splits():
    # int4 tiles pair under several splits only from 64 tiles on: 512 rows after 284
    # tokens (4 before a page boundary), three splits by kvx_prefill_plan
    assert kvx.prefill_plan(284, 512, H, QH, ko.INT4) == 3
    prefill_case(ko.INT4, 284, -512)
    # and under the reference rule's single split for 264 rows, after 1500 tokens
    # (also 4 before a page boundary): the kernel with one register set of pages
    prefill_case(ko.INT4, 1500, 264)


def prefill_case(fmt, committed, rows, forced_splits=None):
    planned, rows = rows < 0, abs(rows)
    tw = Gp.Twin(fmt, H, D, 2, (committed + rows + 31) // 32)
    pages, th, td = fill(tw, committed + rows, seed=committed + rows)
    tw.assert_same_bytes()
    stride = (rows + 31) // 32 * 32
    q = np.zeros((H, stride, G, D), dtype=np.uint16)
    q[:, :rows] = queries((H, rows, G, D), committed)
    splits = kvx.lib().kvx_prefill_splits(rows)
    if planned:
        splits = kvx.prefill_plan(committed, rows, H, QH, fmt)
        assert splits > 1
    if forced_splits:
        splits = forced_splits
    hp = ko.PrefillParams(committed, rows, stride, len(pages), tw.host.layer(1), splits, 0.0)
    ok, want, want32 = ko.attend_prefill(fmt, H, G, D, q, th, hp)
    assert ok == 1
    out = torch.full((H, stride, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.prefill_workspace_bytes(tw.dev, rows, QH, splits), dtype=torch.uint8,
                     device="cuda")
    kvx.attend_prefill(tw.dev, 1, QH, Gp.dev(q), out, td,
                       kvx.PrefillParams(committed, rows, stride, len(pages), kvx.KvLayer(), splits, 0.0), ws)
    torch.cuda.synchronize()
    got = Gp.host_u16(out)
    live = np.zeros((H, stride), dtype=bool)
    live[:, :rows] = True
    stats = Gp.check_attention(got, want, want32, live, tol(fmt),
                               f"prefill fmt={fmt} H={H} G={G} committed={committed} rows={rows}",
                               explain=Gp.prefill_explainer(fmt, H, G, D, q, th, tw.host.layer(1),
                                                            committed, rows, splits))
    # the matrix cores sum in another order than the oracle; the mean stays far
    # below the per-row bar
    assert stats["rel_l2_mean"] < 5e-4
    # rows of the last tile past the chunk are zeros; rows past the tiles are untouched
    tile_end = (rows + 7) // 8 * 8
    assert not got[:, rows:tile_end].any()
    assert (got[:, tile_end:] == 0x5A5A).all()
    tw.close()


@pytest.mark.parametrize("fmt", FORMATS)
def test_verify_chain_matches_oracle(fmt):
    # 348 and 1980 tokens end 4 tokens before a page boundary: the chain's rows see
    # different parts of the last two pages
    committed = [0, 1023, 1023 + 649, 40, 348, 1980]
    lanes = len(committed)
    counts = [(c + 8 + 31) // 32 for c in committed]
    tws, hts, dts = [], [], []
    for lane, c in enumerate(committed):
        tw = Gp.Twin(fmt, H, D, 2, counts[lane])
        pages, th, td = fill(tw, c + 8, seed=300 + lane)
        tws.append(tw)
        hts.append(th)
        dts.append(td)
    # every lane has its own storage here only on the oracle side; the device
    # call needs one storage, so lanes are checked one per call and then batched
    for lane in range(lanes):
        tw = tws[lane]
        q = np.zeros((1, H, 32, G, D), dtype=np.uint16)
        q[:, :, :8] = queries((1, H, 8, G, D), lane)
        splits = kvx.lib().kvx_verify_splits(committed[lane], 8)
        hp = ko.VerifyParams(committed[lane], counts[lane], tw.host.layer(1), splits, 128, 8, 8, 0.0)
        n, want, want32 = ko.attend_verify(fmt, H, G, D, q, [hts[lane]], [hp])
        assert n == 1
        dp = [kvx.VerifyParams(committed[lane], counts[lane], kvx.KvLayer(), splits, splits, 8, 8, 0.0)]
        out = torch.full((1, H, 32, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
        ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
        kvx.attend_verify(tw.dev, 1, QH, Gp.dev(q), out, [dts[lane]], dp, None, 32, ws)
        torch.cuda.synchronize()
        got = Gp.host_u16(out)
        live = np.zeros((1, H, 32), dtype=bool)
        live[:, :, :8] = True
        Gp.check_attention(got, want, want32, live, tol(fmt),
                           f"verify chain fmt={fmt} H={H} G={G} committed={committed[lane]}",
                           explain=Gp.lanes_explainer(fmt, H, G, D, q, [hts[lane]], tw.host.layer(1),
                                                      [committed[lane]], 8, [splits], 8))
        assert (got[:, :, 8:] == 0x5A5A).all()
    for tw in tws:
        tw.close()


def shared_pool_lanes(fmt, committed, rows, seed, layers=2, layer=1):
    """Lanes with their own page tables inside one pool (the batched case)."""
    counts = [(c + rows + 31) // 32 for c in committed]
    tw = Gp.Twin(fmt, H, D, layers, sum(counts))
    ids = tw.pages(sum(counts), seed)
    hts, dts, first = [], [], 0
    rng = np.random.default_rng(seed)
    for lane, n in enumerate(counts):
        th, td = tw.tables(ids[first:first + n])
        first += n
        hts.append(th)
        dts.append(td)
        total = committed[lane] + rows
        done = 0
        while done < total:
            m = min(2048, total - done)
            k = rng.standard_normal((H, m, D)).astype(np.float32)
            v = rng.standard_normal((H, m, D)).astype(np.float32)
            stride = (m + 31) // 32 * 32
            ck, cv = T.chunk_buffers(k, v, stride)
            kvx.append(tw.dev, layer, Gp.dev(ck), Gp.dev(cv), [td],
                       [kvx.ChunkParams(done, m, stride, n)], H * stride * D)
            p = ko.ChunkParams(done, m, stride, n, tw.host.layer(layer))
            assert ko.store_chunk(fmt, H, D, ck, cv, th, p) == 1
            done += m
    torch.cuda.synchronize()
    return tw, counts, hts, dts


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16])
def test_batched_verify_chain_matches_oracle(fmt):
    committed = [0, 1023, 1672, 31, 1980]
    tw, counts, hts, dts = shared_pool_lanes(fmt, committed, 8, seed=41)
    lanes = len(committed)
    q = np.zeros((lanes, H, 32, G, D), dtype=np.uint16)
    q[:, :, :8] = queries((lanes, H, 8, G, D), 5)
    splits = [kvx.lib().kvx_verify_splits(c, 8) for c in committed]
    hp = [ko.VerifyParams(committed[i], counts[i], tw.host.layer(1), splits[i], 128, 8, 8, 0.0)
          for i in range(lanes)]
    n, want, want32 = ko.attend_verify(fmt, H, G, D, q, hts, hp)
    assert n == lanes
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], 128, 8, 8, 0.0)
          for i in range(lanes)]
    out = torch.zeros((lanes, H, 32, G, D), dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
    kvx.attend_verify(tw.dev, 1, QH, Gp.dev(q), out, dts, dp, None, 32, ws)
    torch.cuda.synchronize()
    live = np.zeros((lanes, H, 32), dtype=bool)
    live[:, :, :8] = True
    Gp.check_attention(Gp.host_u16(out), want, want32, live, tol(fmt),
                       f"batched verify chain fmt={fmt} H={H} G={G}",
                       explain=Gp.lanes_explainer(fmt, H, G, D, q, hts, tw.host.layer(1), committed, 8,
                                                  splits, 8))
    # a repeat submission gives the same bits
    out2 = torch.zeros_like(out)
    kvx.attend_verify(tw.dev, 1, QH, Gp.dev(q), out2, dts, dp, None, 32, ws)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    tw.close()


def tree_masks(parents):
    masks = []
    for row, parent in enumerate(parents):
        masks.append((1 << row) | (masks[parent] if parent >= 0 else 0))
    return masks


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16])
@pytest.mark.parametrize("nodes", [15, 16])
def test_tree_verify_matches_oracle(fmt, nodes):
    committed = [260, 31, 4000]
    lanes = len(committed)
    tw, counts, hts, dts = shared_pool_lanes(fmt, committed, nodes, seed=61 + nodes)
    rng = np.random.default_rng(nodes)
    masks = np.zeros((lanes, 16), dtype=np.uint32)
    for lane in range(lanes):
        parents = [-1] + [int(rng.integers(max(0, i - 3), i)) for i in range(1, nodes)]
        masks[lane, :nodes] = tree_masks(parents)
    q = np.zeros((lanes, H, 32, G, D), dtype=np.uint16)
    q[:, :, :16] = queries((lanes, H, 16, G, D), 7)
    splits = [kvx.lib().kvx_verify_splits(c, nodes) for c in committed]
    hp = [ko.VerifyParams(committed[i], counts[i], tw.host.layer(1), splits[i], 128, nodes, 16, 0.0)
          for i in range(lanes)]
    n, want, want32 = ko.attend_verify(fmt, H, G, D, q, hts, hp, masks)
    assert n == lanes
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], 128, nodes, 16, 0.0)
          for i in range(lanes)]
    out = torch.full((lanes, H, 32, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
    kvx.attend_verify(tw.dev, 1, QH, Gp.dev(q), out, dts, dp, Gp.dev(masks), 32, ws)
    torch.cuda.synchronize()
    got = Gp.host_u16(out)
    live = np.zeros((lanes, H, 32), dtype=bool)
    live[:, :, :nodes] = True
    Gp.check_attention(got, want, want32, live, tol(fmt),
                       f"tree verify fmt={fmt} H={H} G={G} nodes={nodes}",
                       explain=Gp.lanes_explainer(fmt, H, G, D, q, hts, tw.host.layer(1), committed,
                                                  nodes, splits, 16, masks))
    assert not got[:, :, nodes:16].any() and (got[:, :, 16:] == 0x5A5A).all()
    tw.close()


@pytest.mark.parametrize("nodes,capacity", [(7, 7), (5, 8)])
def test_int4_small_tree_verify_in_one_wave(nodes, capacity):
    # capacity x group = 42 or 48 fused rows: the int4 kernel that keeps three
    # blocks of 16 fused rows in one wave, with ancestor masks and, for capacity 7,
    # a last block that is only partly in the tile
    fmt = ko.INT4
    committed = [260, 31, 4000, 0]
    lanes = len(committed)
    tw, counts, hts, dts = shared_pool_lanes(fmt, committed, nodes, seed=90 + nodes)
    rng = np.random.default_rng(nodes)
    masks = np.zeros((lanes, capacity), dtype=np.uint32)
    for lane in range(lanes):
        parents = [-1] + [int(rng.integers(max(0, i - 3), i)) for i in range(1, nodes)]
        masks[lane, :nodes] = tree_masks(parents)
    q = np.zeros((lanes, H, 32, G, D), dtype=np.uint16)
    q[:, :, :capacity] = queries((lanes, H, capacity, G, D), 9)
    splits = kvx.verify_plan(committed, nodes, H, QH, fmt)
    splits = [max(s, 2) if c > 64 else s for s, c in zip(splits, committed)]  # merged and single-split lanes
    hp = [ko.VerifyParams(committed[i], counts[i], tw.host.layer(1), splits[i], 128, nodes, capacity, 0.0)
          for i in range(lanes)]
    n, want, want32 = ko.attend_verify(fmt, H, G, D, q, hts, hp, masks)
    assert n == lanes
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], 128, nodes, capacity, 0.0)
          for i in range(lanes)]
    out = torch.full((lanes, H, 32, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
    before = kvx.attend_paths()
    kvx.attend_verify(tw.dev, 1, QH, Gp.dev(q), out, dts, dp, Gp.dev(masks), 32, ws)
    torch.cuda.synchronize()
    after = kvx.attend_paths()
    assert after[1] == before[1] + 1 and after[0] == before[0]  # a matrix-core launch
    got = Gp.host_u16(out)
    live = np.zeros((lanes, H, 32), dtype=bool)
    live[:, :, :nodes] = True
    Gp.check_attention(got, want, want32, live, tol(fmt), f"small tree verify nodes={nodes}",
                       explain=Gp.lanes_explainer(fmt, H, G, D, q, hts, tw.host.layer(1), committed,
                                                  nodes, splits, capacity, masks))
    assert not got[:, :, nodes:capacity].any() and (got[:, :, capacity:] == 0x5A5A).all()
    tw.close()


def decode_case(fmt, committed, seed, row_stride=1, layers=2, layer=1, planned=False):
    lanes = len(committed)
    tw, counts, hts, dts = shared_pool_lanes(fmt, committed, 1, seed=seed, layers=layers, layer=layer)
    q = np.zeros((lanes, H, row_stride, G, D), dtype=np.uint16)
    q[:, :, 0] = queries((lanes, H, G, D), seed)
    splits = (kvx.decode_plan_for(tw.dev, committed) if planned
              else [kvx.lib().kvx_decode_splits(c, 1) for c in committed])
    want = np.zeros((lanes, H, G, D), dtype=np.uint16)
    want32 = np.zeros((lanes, H, G, D), dtype=np.float32)
    for i in range(lanes):
        # the oracle's decode is its prefill entry with one row; its contract
        # bounds the split count at 32, the verify entry at 128
        q1 = np.zeros((1, H, 32, G, D), dtype=np.uint16)
        q1[0, :, 0] = q[i, :, 0]
        hp = ko.VerifyParams(committed[i], counts[i], tw.host.layer(layer), splits[i], 128, 1, 1, 0.0)
        n, o, o32 = ko.attend_verify(fmt, H, G, D, q1, [hts[i]], [hp])
        assert n == 1
        want[i], want32[i] = o[0, :, 0], o32[0, :, 0]
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], splits[i], 1, 1, 0.0)
          for i in range(lanes)]
    out = torch.full((lanes, H, row_stride, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
    kvx.attend_decode(tw.dev, layer, QH, Gp.dev(q), out, dts, dp, row_stride, ws)
    torch.cuda.synchronize()
    got = Gp.host_u16(out)
    stats = Gp.check_attention(got[:, :, 0], want, want32, np.ones((lanes, H), dtype=bool), tol(fmt),
                               f"decode fmt={fmt} H={H} G={G} committed={committed}",
                               explain=Gp.lanes_explainer(fmt, H, G, D, q, hts, tw.host.layer(layer),
                                                          committed, 1, splits, 1, one_row=True))
    assert stats["rel_l2_mean"] < 5e-4
    if row_stride > 1:
        assert (got[:, :, 1:] == 0x5A5A).all()
    tw.close()
    return stats


@pytest.mark.parametrize("fmt", FORMATS)
def test_decode_matches_oracle(fmt):
    decode_case(fmt, [0, 1, 31, 32, 511, 512, 1000, 2047, 4095, 600, 33, 5000], seed=80 + fmt)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("heads,group,dim", [(2, 8, 128), (8, 4, 64)])
def test_decode_under_the_plan_of_its_layout(fmt, heads, group, dim):
    """kvx_decode_plan_for's splits (one round of single waves at head dimensions 64 and 128)
    over ragged lanes, more of them than one launch takes."""
    global H, G, D, QH
    saved = (H, G, D, QH)
    H, G, D, QH = heads, group, dim, heads * group
    try:
        rng = np.random.default_rng(dim + fmt)
        committed = [0, 31, 32, 127, 128, 4095] + [int(x) for x in rng.integers(0, 2500, 30)]
        decode_case(fmt, committed, seed=300 + fmt + dim, planned=True)
    finally:
        H, G, D, QH = saved


@pytest.mark.parametrize("row_stride", [1, 32])
def test_int4_decode_many_lanes_and_strides(row_stride):
    rng = np.random.default_rng(row_stride)
    committed = [int(x) for x in rng.integers(0, 3000, 40)]
    decode_case(ko.INT4, committed, seed=5 + row_stride, row_stride=row_stride)


def test_int4_decode_single_token_is_the_value_row():
    tw, counts, hts, dts = shared_pool_lanes(ko.INT4, [0], 1, seed=3)
    q = queries((1, H, 1, G, D), 1)
    dp = [kvx.VerifyParams(0, 1, kvx.KvLayer(), 1, 1, 1, 1, 0.0)]
    out = torch.zeros((1, H, 1, G, D), dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
    kvx.attend_decode(tw.dev, 1, QH, Gp.dev(q), out, dts, dp, 1, ws)
    torch.cuda.synchronize()
    got = ko.bf16_to_f32(Gp.host_u16(out)).reshape(H, G, D)
    page = int((hts[0][0] & 0x3FFF)) + 0  # index inside its extent
    kc, ks, vc, vs = T.page_codes(tw.host, 1, int(tw.pages(1, 3)[0]))
    for h in range(H):
        w = ko.bf16_to_f32(ko.f32_to_bf16(vs[h, :1]))[0]
        want = ko.bf16_to_f32(ko.f32_to_bf16((w * vc[h, 0]).astype(np.float32)))
        for g in range(G):
            assert np.array_equal(got[h, g], want)
    tw.close()


def test_invalid_attention_parameters_enqueue_nothing():
    tw, counts, hts, dts = shared_pool_lanes(ko.INT8, [40], 8, seed=9)
    q = Gp.dev(queries((1, H, 32, G, D), 2))
    out = torch.full((1, H, 32, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    good = kvx.VerifyParams(40, counts[0], kvx.KvLayer(), 32, 32, 8, 8, 0.0)
    ws = torch.full((kvx.attend_workspace_bytes(tw.dev, [good], QH),), 0xA5, dtype=torch.uint8, device="cuda")
    cases = []
    for field, value in (("page_table_entries", 1), ("split_count", 0), ("split_count", 129),
                         ("active_rows", 0), ("active_rows", 9), ("committed_tokens", 262159),
                         # common/paged_attention_tile.h:57-58: split_count <= slot_splits <= maximum
                         ("slot_splits", 31), ("slot_splits", 129)):
        p = kvx.VerifyParams(40, counts[0], kvx.KvLayer(), 32, 32, 8, 8, 0.0)
        setattr(p, field, value)
        cases.append(p)
    for p in cases:
        with pytest.raises(kvx.KvxError) as err:
            kvx.attend_verify(tw.dev, 1, QH, q, out, dts, [p], None, 32, ws)
        assert err.value.code == kvx.EINVAL
    with pytest.raises(kvx.KvxError):  # undersized scratch
        kvx.attend_verify(tw.dev, 1, QH, q, out, dts, [good], None, 32, ws[:-4])
    with pytest.raises(kvx.KvxError):  # query heads not a multiple of the KV heads
        kvx.attend_verify(tw.dev, 1, QH + 1, q, out, dts, [good], None, 32, ws)
    with pytest.raises(kvx.KvxError):  # aliasing
        kvx.attend_verify(tw.dev, 1, QH, q, q, dts, [good], None, 32, ws)
    bad_prefill = kvx.PrefillParams(40, 8, 32, 1, kvx.KvLayer(), 4, 0.0)
    with pytest.raises(kvx.KvxError):
        kvx.attend_prefill(tw.dev, 1, QH, q, out, dts[0], bad_prefill, ws)
    torch.cuda.synchronize()
    assert (out == 0x5A5A).all() and (ws == 0xA5).all()
    tw.close()


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("heads,group,dim", [(2, 3, 128), (4, 6, 128), (3, 2, 64), (2, 8, 128), (8, 4, 64),
                                              (1, 20, 256)])
def test_generic_kernels_cover_other_shapes(fmt, heads, group, dim):
    """Head dimensions other than 256: chunked prefill, chain verify and decode.  64 and 128
    (the reference's other layouts, 2 x 8 x 128 and 8 x 4 x 64 among them) run the tile on the
    matrix cores out of a staged copy of the page; anything else (here a group of 20 query
    heads, whose tiles of 8 rows would exceed 128 fused rows: verify of 6 rows and decode only)
    runs on the format-generic kernels, which keep the oracle's operation order (nearly every
    output has the oracle's bits)."""
    in_order = dim not in (64, 128)
    committed, rows = 300, 13
    tw = Gp.Twin(fmt, heads, dim, 2, (committed + rows + 31) // 32)
    pages, th, td = fill(tw, committed + rows, seed=dim + heads)
    tw.assert_same_bytes()
    qh = heads * group
    chain = min(8, 128 // group)
    # prefill (a tile is 8 rows x group fused rows, 128 at most)
    if 8 * group <= 128:
        q = np.zeros((heads, 32, group, dim), dtype=np.uint16)
        q[:, :rows] = queries((heads, rows, group, dim), dim)
        splits = kvx.lib().kvx_prefill_splits(rows)
        hp = ko.PrefillParams(committed, rows, 32, len(pages), tw.host.layer(1), splits, 0.0)
        ok, want, want32 = ko.attend_prefill(fmt, heads, group, dim, q, th, hp)
        assert ok == 1
        out = torch.zeros((heads, 32, group, dim), dtype=torch.int16, device="cuda")
        ws = torch.empty(kvx.prefill_workspace_bytes(tw.dev, rows, qh), dtype=torch.uint8, device="cuda")
        kvx.attend_prefill(tw.dev, 1, qh, Gp.dev(q), out, td,
                           kvx.PrefillParams(committed, rows, 32, len(pages), kvx.KvLayer(), splits, 0.0), ws)
        torch.cuda.synchronize()
        live = np.zeros((heads, 32), dtype=bool)
        live[:, :rows] = True
        stats = Gp.check_attention(Gp.host_u16(out), want, want32, live, tol(fmt), f"generic prefill {fmt}",
                                   explain=None if in_order else Gp.prefill_explainer(
                                       fmt, heads, group, dim, q, th, tw.host.layer(1), committed, rows, splits))
        assert stats["exact"] > 0.98 or not in_order
        assert stats["rel_l2_mean"] < 5e-4
    # chain verify of 8 rows (6 for the group of 20) and one-row decode over the same pages
    for active, capacity, row_stride in ((chain, chain, 32), (1, 1, 1)):
        visible = committed + active
        q = np.zeros((1, heads, row_stride, group, dim), dtype=np.uint16)
        q[:, :, :active] = queries((1, heads, active, group, dim), active)
        splits = (kvx.lib().kvx_verify_splits(committed, active) if capacity > 1
                  else max(2, kvx.lib().kvx_decode_splits(committed, 1)))
        hp = ko.VerifyParams(committed, len(pages), tw.host.layer(1), splits, 128, active, capacity, 0.0)
        qo = q if capacity > 1 else np.concatenate(
            [q, np.zeros((1, heads, 31, group, dim), dtype=np.uint16)], axis=2)
        n, want, want32 = ko.attend_verify(fmt, heads, group, dim, qo, [th], [hp])
        assert n == 1 and visible <= committed + rows
        dp = [kvx.VerifyParams(committed, len(pages), kvx.KvLayer(), splits, splits, active, capacity, 0.0)]
        out = torch.zeros((1, heads, row_stride, group, dim), dtype=torch.int16, device="cuda")
        ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, qh), dtype=torch.uint8, device="cuda")
        if capacity > 1:
            kvx.attend_verify(tw.dev, 1, qh, Gp.dev(q), out, [td], dp, None, row_stride, ws)
        else:
            kvx.attend_decode(tw.dev, 1, qh, Gp.dev(q), out, [td], dp, row_stride, ws)
        torch.cuda.synchronize()
        live = np.zeros((1, heads, row_stride), dtype=bool)
        live[:, :, :active] = True
        Gp.check_attention(Gp.host_u16(out), want[:, :, :row_stride], want32[:, :, :row_stride], live,
                           tol(fmt), f"generic rows={active} fmt={fmt}",
                           explain=None if in_order else Gp.lanes_explainer(
                               fmt, heads, group, dim, qo, [th], tw.host.layer(1), [committed], [active],
                               [splits], capacity))
    tw.close()


@pytest.mark.parametrize("fmt", FORMATS)
def test_append_attend_decode_is_the_two_calls(fmt):
    """kv_append_attend_decode leaves the page bytes of kv_append (the oracle's,
    bit for bit) and returns the output of kv_attend_decode; int4 pages take the
    kernel that stores the token itself."""
    committed = [0, 31, 32, 700, 4095, 1000, 63, 2047, 5000]
    if fmt == ko.INT4:  # more lanes than one launch holds
        committed += [int(x) for x in np.random.default_rng(60).integers(0, 1500, 31)]
    lanes = len(committed)
    tw, counts, hts, dts = shared_pool_lanes(fmt, committed, 1, seed=61)
    rng = np.random.default_rng(62)
    k = rng.standard_normal((lanes, H, 1, D)).astype(np.float32)
    v = rng.standard_normal((lanes, H, 1, D)).astype(np.float32)
    k[:, :, :, [3, 77]] *= 20
    k[2, 1] = 0  # a zero row: scale 0, codes 0
    v[5, H - 1] *= 1e-20
    ck = np.zeros((lanes, H, 32, D), dtype=np.uint16)
    cv = np.zeros((lanes, H, D, 32), dtype=np.uint16)
    for lane in range(lanes):
        ck[lane], cv[lane] = T.chunk_buffers(k[lane], v[lane], 32)
    q = queries((lanes, H, 1, G, D), 63)
    splits = [max(kvx.lib().kvx_decode_splits(c, 1), 1 + (c > 600)) for c in committed]
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], splits[i], 1, 1, 0.0)
          for i in range(lanes)]
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
    before = [tw.dev.extent_read(e).copy() for e in range(tw.extents)]
    # the two calls
    kvx.append(tw.dev, 1, Gp.dev(ck), Gp.dev(cv), dts,
               [kvx.ChunkParams(committed[i], 1, 32, counts[i]) for i in range(lanes)], H * 32 * D)
    out_two = torch.zeros((lanes, H, 1, G, D), dtype=torch.int16, device="cuda")
    kvx.attend_decode(tw.dev, 1, QH, Gp.dev(q), out_two, dts, dp, 1, ws)
    torch.cuda.synchronize()
    for lane in range(lanes):
        p = ko.ChunkParams(committed[lane], 1, 32, counts[lane], tw.host.layer(1))
        assert ko.store_chunk(fmt, H, D, ck[lane], cv[lane], hts[lane], p) == 1
    tw.assert_same_bytes()
    # back to the state before the step, then the one call
    for e in range(tw.extents):
        tw.dev.extent_write(e, before[e])
    out_one = torch.zeros_like(out_two)
    ws.fill_(0xA5)
    kvx.append_attend_decode(tw.dev, 1, Gp.dev(ck), Gp.dev(cv), H * 32 * D, 32, QH, Gp.dev(q), out_one,
                             dts, dp, 1, ws)
    torch.cuda.synchronize()
    tw.assert_same_bytes()
    assert torch.equal(out_one, out_two)
    # and its parameter checks
    with pytest.raises(kvx.KvxError):
        kvx.append_attend_decode(tw.dev, 1, Gp.dev(ck), Gp.dev(cv), H * 32 * D, 31, QH, Gp.dev(q),
                                 out_one, dts, dp, 1, ws)
    tw.close()


@pytest.mark.parametrize("fmt", FORMATS)
def test_rows_of_a_single_token_have_the_oracles_bits(fmt):
    single_token_rows(fmt, H, G, D)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("heads,group,dim", [(4, 4, 128), (8, 4, 64)])
def test_rows_of_a_single_token_at_other_head_dimensions(fmt, heads, group, dim):
    single_token_rows(fmt, heads, group, dim)


def single_token_rows(fmt, heads, group, dim):
    """A sequence of one token: its weight is exp(score - score) = 1 and every output element is
    one product, often a tie between two bf16 values (an 8-bit weight times a small code), so the
    output must be the oracle's bit for bit.  A product fused into the difference behind it (score
    = dot x scale, then score - maximum) leaves the product's rounding error in place of zero, a
    weight of 0.99999994, and every tie falls the other way: found by a seeded search at head
    dimension 128, where the statistics of such a row read (score, 0.99999994)."""
    lanes = 12
    tw = Gp.Twin(fmt, heads, dim, 2, lanes)
    ids = tw.pages(lanes, 5)
    rng = np.random.default_rng(11 + dim)
    hts, dts = [], []
    for lane in range(lanes):
        th, td = tw.tables(ids[lane:lane + 1])
        hts.append(th)
        dts.append(td)
        k = rng.standard_normal((heads, 1, dim)).astype(np.float32)
        v = rng.standard_normal((heads, 1, dim)).astype(np.float32)
        ck, cv = T.chunk_buffers(k, v, 32)
        kvx.append(tw.dev, 1, Gp.dev(ck), Gp.dev(cv), [td], [kvx.ChunkParams(0, 1, 32, 1)], heads * 32 * dim)
        assert ko.store_chunk(fmt, heads, dim, ck, cv, th, ko.ChunkParams(0, 1, 32, 1, tw.host.layer(1))) == 1
    qh = heads * group
    q = np.zeros((lanes, heads, 1, group, dim), dtype=np.uint16)
    q[:, :, 0] = queries((lanes, heads, group, dim), 12)
    want = np.zeros((lanes, heads, group, dim), dtype=np.uint16)
    for i in range(lanes):
        q1 = np.zeros((1, heads, 32, group, dim), dtype=np.uint16)
        q1[0, :, 0] = q[i, :, 0]
        n, o, _ = ko.attend_verify(fmt, heads, group, dim, q1, [hts[i]],
                                   [ko.VerifyParams(0, 1, tw.host.layer(1), 1, 128, 1, 1, 0.0)])
        assert n == 1
        want[i] = o[0, :, 0]
    dp = [kvx.VerifyParams(0, 1, kvx.KvLayer(), 1, 1, 1, 1, 0.0) for _ in range(lanes)]
    out = torch.zeros((lanes, heads, 1, group, dim), dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, qh) + 256, dtype=torch.uint8, device="cuda")
    kvx.attend_decode(tw.dev, 1, qh, Gp.dev(q), out, dts, dp, 1, ws)
    # the same rows as partial rows: the sum of a single weight is 1, to the bit
    total = lanes * heads * group
    statistics_at = (total * dim * 4 + 255) // 256 * 256
    ws2 = torch.zeros(statistics_at + total * 8 + 256, dtype=torch.uint8, device="cuda")
    kvx.attend_split(tw.dev, 1, qh, Gp.dev(q), dts, dp, None, 1, ws2)
    torch.cuda.synchronize()
    sums = ws2[statistics_at:statistics_at + total * 8].cpu().numpy().view(np.float32).reshape(total, 2)[:, 1]
    assert (sums == np.float32(1.0)).all(), sums[sums != 1.0][:4]
    assert np.array_equal(Gp.host_u16(out)[:, :, 0], want)
    tw.close()
