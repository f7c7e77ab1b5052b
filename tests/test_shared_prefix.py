"""One-row decode attention of sequences that share their first pages
(kv_attend_decode_shared): the shared pages are read once for all of them.

The reference has no such kernel (it lists the case as a gap).  The oracle here is
built from the reference's own pieces in the same arrangement: its attention tile
over the shared pages for the stacked rows, its tile over each sequence's own
pages, and its fixed-order merge over both lists of splits.  Against that the bar
is the attention bar of the other tests (relative L2 per output row <= 2e-3).

Against the ordinary decode of every sequence over its whole page table the
agreement is looser by construction, and the test says so: probabilities are
rounded to bf16 relative to the running maximum of their split (P = bf16(p x value
scale), the reference's rule), so another partition into splits rounds every
probability differently; on random values those roundings do not average out (the
output is itself a sum of as many random terms), which leaves about 1.5e-3 between
any two partitions, the oracle's own included, and up to 4.5e-3 on sequences of under a
hundred tokens (a seeded search over random shapes: int8 pages, a prefix of one or two pages;
the oracle's two arrangements lay exactly as far apart as the library's).  So the library is
held to the oracle's own distance between the two arrangements, row by row, plus the bar.
"""
import numpy as np
import pytest

from oracle import kvoracle as ko
from richengine_amd import kvx
import kvtestlib as T

pytestmark = pytest.mark.gpu
H, G, D = 4, 6, 256
QH = H * G


def shared_pool(fmt, shared_pages, own_tokens, seed, layer=1):
    """Sequences whose tables begin with the same `shared_pages` pages; own_tokens[i] tokens of
    sequence i follow the prefix.  Filled on the device, mirrored into the oracle store."""
    import torch
    import gpulib as Gp
    lanes = len(own_tokens)
    own_pages = [(t + 1 + 31) // 32 for t in own_tokens]
    tw = Gp.Twin(fmt, H, D, 2, shared_pages + sum(own_pages))
    ids = tw.pages(shared_pages + sum(own_pages), seed)
    prefix = ids[:shared_pages]
    rng = np.random.default_rng(seed)
    hts, dts, first = [], [], shared_pages
    for n in own_pages:
        th, td = tw.tables(np.concatenate([prefix, ids[first:first + n]]))
        first += n
        hts.append(th)
        dts.append(td)

    def fill(lane, start, count):
        done = 0
        while done < count:
            m = min(2048, count - done)
            k = rng.standard_normal((H, m, D)).astype(np.float32)
            v = rng.standard_normal((H, m, D)).astype(np.float32)
            stride = (m + 31) // 32 * 32
            ck, cv = T.chunk_buffers(k, v, stride)
            entries = shared_pages + own_pages[lane]
            kvx.append(tw.dev, layer, Gp.dev(ck), Gp.dev(cv), [dts[lane]],
                       [kvx.ChunkParams(start + done, m, stride, entries)], H * stride * D)
            p = ko.ChunkParams(start + done, m, stride, entries, tw.host.layer(layer))
            assert ko.store_chunk(fmt, H, D, ck, cv, hts[lane], p) == 1
            done += m

    fill(0, 0, shared_pages * 32)  # the prefix, once, through the first sequence's table
    for lane in range(lanes):
        fill(lane, shared_pages * 32, own_tokens[lane] + 1)  # its own tokens and the step's token
    torch.cuda.synchronize()
    tw.assert_same_bytes()
    return tw, hts, dts, [shared_pages + n for n in own_pages]


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16])
@pytest.mark.parametrize("shared_pages,own_tokens,prefix_splits", [
    (40, [0, 5, 31, 32, 700, 64, 1], 5),      # 7 sequences: 42 fused rows over the prefix
    (3, [10, 2000], 1),                      # 12 fused rows: the one-block kernel; a single prefix split
    (129, [3] * 16, 16),                     # 16 sequences, 96 fused rows
])
def test_shared_prefix_decode_matches_oracle(fmt, shared_pages, own_tokens, prefix_splits):
    import torch
    import gpulib as Gp
    import test_gpu_attention as A
    lanes = len(own_tokens)
    tw, hts, dts, entries = shared_pool(fmt, shared_pages, own_tokens, seed=300 + shared_pages)
    committed = [shared_pages * 32 + t for t in own_tokens]
    q = A.queries((lanes, H, 1, G, D), 17)
    want = np.zeros((lanes, H, G, D), dtype=np.uint16)
    want32 = np.zeros((lanes, H, G, D), dtype=np.float32)
    for i in range(lanes):
        q1 = np.zeros((1, H, 32, G, D), dtype=np.uint16)
        q1[0, :, 0] = q[i, :, 0]
        splits = kvx.lib().kvx_decode_splits(committed[i], 1)
        hp = ko.VerifyParams(committed[i], entries[i], tw.host.layer(1), splits, 128, 1, 1, 0.0)
        n, o, o32 = ko.attend_verify(fmt, H, G, D, q1, [hts[i]], [hp])
        assert n == 1
        want[i], want32[i] = o[0, :, 0], o32[0, :, 0]
    own_splits = [max(1, -(-((t + 1 + 31) // 32) // 8)) for t in own_tokens]
    dp = [kvx.VerifyParams(committed[i], entries[i], kvx.KvLayer(), own_splits[i], own_splits[i], 1, 1, 0.0)
          for i in range(lanes)]
    ws = torch.empty(kvx.attend_shared_workspace_bytes(tw.dev, dp, prefix_splits, QH), dtype=torch.uint8,
                     device="cuda")
    out = torch.full((lanes, H, 1, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    kvx.attend_decode_shared(tw.dev, 1, QH, Gp.dev(q), out, dts, dp, shared_pages, prefix_splits, 1, ws)
    torch.cuda.synchronize()
    got = Gp.host_u16(out)[:, :, 0]
    same, same32 = oracle_shared(fmt, tw, hts, entries, q, shared_pages, own_tokens, prefix_splits, own_splits)
    Gp.check_attention(got, same, same32, np.ones((lanes, H), dtype=bool), A.tol(fmt),
                       f"shared prefix fmt={fmt} pages={shared_pages}",
                       explain=lambda index: dict(rows=flipped_rows(
                           fmt, tw, hts, entries, q, shared_pages, own_tokens, prefix_splits, own_splits,
                           committed, index)))
    # the ordinary decode of every sequence, another partition: see the module's note
    value = lambda bits: ko.bf16_to_f32(bits).reshape(bits.shape).astype(np.float64)
    apart = np.linalg.norm(value(got) - value(want), axis=-1) / np.linalg.norm(value(want), axis=-1)
    between = np.linalg.norm(value(same) - value(want), axis=-1) / np.linalg.norm(value(want), axis=-1)
    # no farther from the ordinary decode than the oracle's own shared arrangement is, plus the bar
    assert (apart <= between + A.tol(fmt)).all(), (apart.max(), between.max())
    # the unshared entry over the same tables
    plain = torch.zeros_like(out)
    up = [kvx.VerifyParams(committed[i], entries[i], kvx.KvLayer(), kvx.lib().kvx_decode_splits(committed[i], 1),
                           128, 1, 1, 0.0) for i in range(lanes)]
    ws2 = torch.empty(kvx.attend_workspace_bytes(tw.dev, up, QH), dtype=torch.uint8, device="cuda")
    kvx.attend_decode(tw.dev, 1, QH, Gp.dev(q), plain, dts, up, 1, ws2)
    torch.cuda.synchronize()
    a = ko.bf16_to_f32(got).reshape(got.shape).astype(np.float64)
    b = ko.bf16_to_f32(Gp.host_u16(plain)[:, :, 0]).reshape(got.shape).astype(np.float64)
    relative = np.linalg.norm(a - b, axis=-1) / np.linalg.norm(b, axis=-1)
    assert (relative <= between + 2 * A.tol(fmt)).all(), (relative.max(), between.max())
    # the same call again gives the same bits
    again = torch.zeros_like(out)
    kvx.attend_decode_shared(tw.dev, 1, QH, Gp.dev(q), again, dts, dp, shared_pages, prefix_splits, 1, ws)
    torch.cuda.synchronize()
    assert torch.equal(out, again)
    tw.close()


def flipped_rows(fmt, tw, hts, entries, q, shared_pages, own_tokens, prefix_splits, own_splits,
                 committed, index, layer=1, top=32, together=2):
    """For check_attention's allowance: output row (lane, head, head in group) in the shared
    arrangement with the roundings turned of those of its heaviest tokens whose weights sit on a
    rounding boundary (ko.rounding_flip_rows says how close), the tokens being in the prefix tile
    or in the sequence's own."""
    import itertools
    lane, head, g = index
    weights = np.zeros(committed[lane] + 1, dtype=np.float32)
    ko.lib().ko_attention_row_weights(fmt, H, D, ko.ptr(np.ascontiguousarray(q[lane, head, 0, g])),
                                      ko.ptr(hts[lane]), tw.host.layer(layer), head, committed[lane], 1,
                                      0, None, 0.0, ko.ptr(weights))
    heaviest = [int(t) for t in np.argsort(-weights, kind="stable")[:top]]

    def recompute(tokens):
        return oracle_shared(fmt, tw, hts, entries, q, shared_pages, own_tokens, prefix_splits,
                             own_splits, layer, only=index, flips=tokens)

    _, _, applied = recompute(heaviest)
    near = [t for t in heaviest if t in applied]
    for size in range(1, min(together, len(near)) + 1):
        for tokens in itertools.combinations(near, size):
            bits, _, _ = recompute(list(tokens))
            yield tokens, size, bits[lane, head, g]


def oracle_shared(fmt, tw, hts, entries, q, shared_pages, own_tokens, prefix_splits, own_splits, layer=1,
                  only=None, flips=None):
    """The oracle's tiles in the shared arrangement, merged in the library's order.  only =
    (lane, head, head in group): that output row alone; flips = tokens of that sequence whose
    roundings are turned where they sit on a boundary (ko_attention_flips), in which case the
    tokens that were turned are returned as a third value."""
    L = ko.lib()
    lanes = len(own_tokens)
    kv = tw.host.layer(layer)
    f32 = np.float32

    def written(tokens, splits):
        pages = (tokens + 31) // 32
        per = -(-pages // splits)
        return -(-pages // per)

    def tiles(queries, table, committed, active, capacity, splits, masks, head, moved=None):
        M = capacity * G
        partials = np.zeros((splits, M, D), dtype=np.float32)
        statistics = np.zeros((splits, M, 2), dtype=np.float32)
        tile_q = np.ascontiguousarray(queries, dtype=np.uint16).reshape(M, D)
        if moved:
            arr = np.array(moved[1], dtype=np.uint32)
            L.ko_attention_flips(moved[0], ko.ptr(arr) if len(arr) else None, len(arr), ko.flip_slack(fmt), 1)
        try:
            for split in range(splits):
                L.ko_attention_tile(fmt, H, G, D, capacity, ko.ptr(tile_q), ko.ptr(table), kv, head,
                                    committed, active, splits, split, ko.ptr(partials),
                                    ko.ptr(statistics), split,
                                    ko.ptr(masks) if masks is not None else None, 0.0)
            if moved:
                mask = L.ko_attention_flips_applied()
                turned.update(moved[2] + t for i, t in enumerate(moved[1]) if mask >> i & 1)
        finally:
            L.ko_attention_flips(-1, None, 0, 0.0, 0)
        return partials, statistics

    out = np.zeros((lanes, H, G, D), dtype=np.float32)
    turned = set()
    zero_masks = np.zeros(lanes, dtype=np.uint32)
    shared_tokens = shared_pages * 32
    for head in range(H) if only is None else [only[1]]:
        # a moved weight sits in one of the two tiles; with `only`, each tile computes one row
        # (fused row, tokens of the tile, what to add to name them as tokens of the sequence)
        in_prefix = in_own = None
        if only is not None:
            mine = flips or []
            in_prefix = (only[0] * G + only[2], [t for t in mine if t < shared_tokens], 0)
            in_own = (only[2], [t - shared_tokens for t in mine if t >= shared_tokens], shared_tokens)
        pp, ps = tiles(q[:, head, 0], hts[0], shared_tokens, lanes, lanes, prefix_splits, zero_masks, head,
                       in_prefix)
        pw = written(shared_tokens + lanes, prefix_splits)
        for i in range(lanes) if only is None else [only[0]]:
            own_table = np.ascontiguousarray(hts[i][shared_pages:])
            op, os_ = tiles(q[i, head, 0], own_table, own_tokens[i], 1, 1, own_splits[i], None, head, in_own)
            ow = written(own_tokens[i] + 1, own_splits[i])
            for g in range(G) if only is None else [only[2]]:
                rows = [(pp[k, i * G + g], ps[k, i * G + g]) for k in range(pw)]
                rows += [(op[k, g], os_[k, g]) for k in range(ow)]
                maximum = max(st[0] for _, st in rows)
                numerator, denominator = np.zeros(D, dtype=f32), f32(0)
                for part, st in rows:
                    weight = np.exp(f32(st[0]) - f32(maximum), dtype=f32) if np.isfinite(st[0]) else f32(0)
                    numerator = numerator + weight * part
                    denominator = f32(denominator + weight * f32(st[1]))
                out[i, head, g] = numerator / denominator
    if flips is not None:
        return ko.f32_to_bf16(out).reshape(out.shape), out, turned
    return ko.f32_to_bf16(out).reshape(out.shape), out


def test_shared_prefix_rejects_bad_arguments():
    import torch
    import gpulib as Gp
    tw, hts, dts, entries = shared_pool(ko.INT4, 2, [5, 40], seed=9)
    committed = [64 + 5, 64 + 40]
    dp = [kvx.VerifyParams(committed[i], entries[i], kvx.KvLayer(), 1, 1, 1, 1, 0.0) for i in range(2)]
    q = torch.zeros((2, H, 1, G, D), dtype=torch.int16, device="cuda")
    out = torch.full((2, H, 1, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_shared_workspace_bytes(tw.dev, dp, 1, QH), dtype=torch.uint8, device="cuda")
    inside = [kvx.VerifyParams(40, entries[0], kvx.KvLayer(), 1, 1, 1, 1, 0.0), dp[1]]
    scaled = [dp[0], kvx.VerifyParams(committed[1], entries[1], kvx.KvLayer(), 1, 1, 1, 1, 0.5)]
    for lanes, shared, splits, space in ((dp, 0, 1, ws), (dp, 2, 0, ws), (dp, 2, 129, ws), (inside, 2, 1, ws),
                                         (scaled, 2, 1, ws), (dp, 2, 1, ws[:1024])):
        with pytest.raises(kvx.KvxError) as e:
            kvx.attend_decode_shared(tw.dev, 1, QH, q, out, dts, lanes, shared, splits, 1, space)
        assert e.value.code == kvx.EINVAL
    torch.cuda.synchronize()
    assert (out == 0x5A5A).all()
    tw.close()
