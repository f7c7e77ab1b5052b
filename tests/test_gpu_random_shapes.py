"""Seeded random shapes of verify and decode batches against the oracle: lane counts on both
sides of what one launch takes, ragged contexts from empty to a few thousand tokens, chains and
trees of 1 to 16 rows with any row capacity, split counts from the reference's rule, from the
plans and drawn at random.  The named cases elsewhere each hold one kernel path to the oracle;
these walk the combinations between them (which kernel a shape selects, lanes with one split next
to lanes with many, launches that mix both), to the same per-row bar."""
import numpy as np
import pytest
import torch

from oracle import kvoracle as ko
from richengine_amd import kvx
import gpulib as Gp
from test_gpu_attention import H, G, D, QH, queries, shared_pool_lanes, tol, tree_masks

pytestmark = pytest.mark.gpu
FORMATS = [ko.INT4, ko.INT8, ko.BF16, ko.FP8]


def draw_contexts(rng, lanes, budget):
    """Ragged contexts: some empty or tiny, some at page boundaries, the rest up to `budget`
    tokens in all."""
    most = max(64, budget // lanes)
    out = []
    for _ in range(lanes):
        kind = rng.integers(0, 6)
        if kind == 0:
            out.append(int(rng.integers(0, 3)))
        elif kind == 1:
            out.append(int(32 * rng.integers(0, most // 32 + 1) + rng.choice([-1, 0, 1]) % 32))
        else:
            out.append(int(rng.integers(0, most)))
    return out


def draw_splits(rng, committed, rows, fmt, decode):
    pages = [(c + rows + 31) // 32 for c in committed]
    kind = rng.integers(0, 3)
    if kind == 0:     # the reference's rule
        if decode:
            return [int(kvx.lib().kvx_decode_splits(c, 1)) for c in committed]
        return [int(kvx.lib().kvx_verify_splits(c, rows)) for c in committed]
    if kind == 1:     # the plans
        return kvx.decode_plan(committed, H, fmt) if decode else kvx.verify_plan(committed, rows, H, QH, fmt)
    return [int(rng.integers(1, min(128, max(1, 2 * n)) + 1)) for n in pages]   # anything valid


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("case", range(5))
def test_random_verify_batches_match_oracle(fmt, case):
    if fmt == ko.FP8 and case >= 3:
        pytest.skip("the fp8 tile has no tree variant; three chain cases")
    rng = np.random.default_rng(1000 * fmt + case)
    lanes = int(rng.choice([1, 2, 3, 5, 8, 33, 36])) if case else 34
    rows = int(rng.integers(1, 17))
    capacity = int(rng.integers(rows, 17))
    tree = fmt != ko.FP8 and bool(rng.integers(0, 2))
    committed = draw_contexts(rng, lanes, 14000)
    splits = draw_splits(rng, committed, rows, fmt, decode=False)
    tw, counts, hts, dts = shared_pool_lanes(fmt, committed, rows, seed=7000 + 10 * fmt + case)
    masks = None
    if tree:
        masks = np.zeros((lanes, capacity), dtype=np.uint32)
        for lane in range(lanes):
            parents = [-1] + [int(rng.integers(max(0, i - 3), i)) for i in range(1, rows)]
            masks[lane, :rows] = tree_masks(parents)
    q = np.zeros((lanes, H, 32, G, D), dtype=np.uint16)
    q[:, :, :capacity] = queries((lanes, H, capacity, G, D), case)
    slot = [int(rng.choice([s, 128])) for s in splits]
    hp = [ko.VerifyParams(committed[i], counts[i], tw.host.layer(1), splits[i], slot[i], rows, capacity, 0.0)
          for i in range(lanes)]
    n, want, want32 = ko.attend_verify(fmt, H, G, D, q, hts, hp, masks)
    assert n == lanes
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], slot[i], rows, capacity, 0.0)
          for i in range(lanes)]
    out = torch.full((lanes, H, 32, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
    what = (f"random verify fmt={fmt} case={case} lanes={lanes} rows={rows}/{capacity} tree={tree} "
            f"committed={committed} splits={splits}")
    print(what, flush=True)
    kvx.attend_verify(tw.dev, 1, QH, Gp.dev(q), out, dts, dp, None if masks is None else Gp.dev(masks), 32, ws)
    torch.cuda.synchronize()
    got = Gp.host_u16(out)
    live = np.zeros((lanes, H, 32), dtype=bool)
    live[:, :, :rows] = True
    Gp.check_attention(got, want, want32, live, tol(fmt), what,
                       explain=Gp.lanes_explainer(fmt, H, G, D, q, hts, tw.host.layer(1), committed, rows,
                                                  splits, capacity, masks))
    assert not got[:, :, rows:capacity].any() and (got[:, :, capacity:] == 0x5A5A).all()
    tw.close()


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("case", range(3))
def test_random_decode_batches_match_oracle(fmt, case):
    rng = np.random.default_rng(2000 * fmt + case)
    lanes = int(rng.choice([1, 4, 31, 32, 33, 47]))
    row_stride = int(rng.choice([1, 2, 32]))
    committed = draw_contexts(rng, lanes, 30000)
    splits = draw_splits(rng, committed, 1, fmt, decode=True)
    tw, counts, hts, dts = shared_pool_lanes(fmt, committed, 1, seed=9000 + 10 * fmt + case)
    q = np.zeros((lanes, H, row_stride, G, D), dtype=np.uint16)
    q[:, :, 0] = queries((lanes, H, G, D), 50 + case)
    want = np.zeros((lanes, H, G, D), dtype=np.uint16)
    want32 = np.zeros((lanes, H, G, D), dtype=np.float32)
    for i in range(lanes):
        q1 = np.zeros((1, H, 32, G, D), dtype=np.uint16)
        q1[0, :, 0] = q[i, :, 0]
        hp = ko.VerifyParams(committed[i], counts[i], tw.host.layer(1), splits[i], max(128, splits[i]), 1, 1, 0.0)
        n, o, o32 = ko.attend_verify(fmt, H, G, D, q1, [hts[i]], [hp])
        assert n == 1
        want[i], want32[i] = o[0, :, 0], o32[0, :, 0]
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], splits[i], 1, 1, 0.0)
          for i in range(lanes)]
    out = torch.full((lanes, H, row_stride, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")
    what = f"random decode fmt={fmt} case={case} lanes={lanes} stride={row_stride} committed={committed} splits={splits}"
    print(what, flush=True)
    kvx.attend_decode(tw.dev, 1, QH, Gp.dev(q), out, dts, dp, row_stride, ws)
    torch.cuda.synchronize()
    got = Gp.host_u16(out)
    Gp.check_attention(got[:, :, 0], want, want32, np.ones((lanes, H), dtype=bool), tol(fmt), what,
                       explain=Gp.lanes_explainer(fmt, H, G, D, q, hts, tw.host.layer(1), committed, 1,
                                                  splits, 1, one_row=True))
    if row_stride > 1:
        assert (got[:, :, 1:] == 0x5A5A).all()
    tw.close()


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("case", range(4))
def test_random_prefill_chunks_match_oracle(fmt, case):
    from test_gpu_attention import prefill_case
    rng = np.random.default_rng(3000 * fmt + case)
    committed = int(rng.choice([0, int(rng.integers(0, 64)), 32 * int(rng.integers(0, 60)),
                                int(rng.integers(0, 2500))]))
    rows = int(rng.choice([int(rng.integers(1, 9)), int(rng.integers(9, 80)), int(rng.integers(80, 400))]))
    kind = rng.integers(0, 3)
    splits = (int(kvx.lib().kvx_prefill_splits(rows)) if kind == 0 else
              kvx.prefill_plan(committed, rows, H, QH, fmt) if kind == 1 else int(rng.integers(1, 33)))
    print(f"random prefill fmt={fmt} case={case} committed={committed} rows={rows} splits={splits}", flush=True)
    prefill_case(fmt, committed, rows, forced_splits=splits)


def test_row_moved_by_a_token_past_its_thirty_two_heaviest():
    """A seed this file's search turned up: 36 int8 lanes of 12-row trees, where one row over 150
    tokens lies 2.1e-3 from the oracle because its 40th heaviest token (weight 8.4e-3, 1.1e-7 from a
    tie between two bf16 values) was rounded the other way: exactly one place of that weight in one
    split's partial row, every other split's partial row bit-equal.  The proof of a turned rounding
    has to reach that far down the row's tokens."""
    test_random_verify_batches_match_oracle(ko.INT8, 31)
