"""kv_attend_prefill_batch: the chunks of several sequences in one call.  Every sequence's rows
must be the bits kv_attend_prefill gives for that sequence alone (which the other tests hold to
the oracle), whether the chunks share their launches (equal shapes) or run one after the other."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

import gpulib as Gp  # noqa: E402
from oracle import kvoracle as ko  # noqa: E402
from richengine_amd import kvx  # noqa: E402
from test_gpu_attention import fill, queries  # noqa: E402

H, G, D = 4, 6, 256
QH = H * G
FORMATS = [ko.INT4, ko.INT8, ko.BF16, ko.FP8]


def run_batch(fmt, committed, rows, splits, poison=0x5A5A):
    """Fills one history per sequence, runs the batch call and every sequence alone; returns
    (batch rows, rows alone, the twin to close)."""
    n = len(committed)
    tokens = [c + r for c, r in zip(committed, rows)]
    counts = [(t + 31) // 32 for t in tokens]
    tw = Gp.Twin(fmt, H, D, 2, sum(counts))
    drawn = tw.pages(sum(counts), seed=sum(tokens))   # no page in two sequences
    strides = [(r + 31) // 32 * 32 for r in rows]
    sequence_stride = H * max(strides) * G * D
    q = np.zeros((n, sequence_stride), dtype=np.uint16)
    tables, params = [], []
    for i in range(n):
        pages, th, td = fill(tw, tokens[i], seed=17 * i + tokens[i],
                             pages=drawn[sum(counts[:i]):sum(counts[:i + 1])])
        qi = np.zeros((H, strides[i], G, D), dtype=np.uint16)
        qi[:, :rows[i]] = queries((H, rows[i], G, D), 31 * i + committed[i])
        q[i, :qi.size] = qi.ravel()
        tables.append(td)
        params.append(kvx.PrefillParams(committed[i], rows[i], strides[i], len(pages), kvx.KvLayer(),
                                        splits[i], 0.0))
    dq = Gp.dev(q)
    bound = sum(kvx.prefill_workspace_bytes(tw.dev, rows[i], QH, splits[i]) for i in range(n)) + 256
    ws = torch.empty(bound, dtype=torch.uint8, device="cuda")
    together = torch.full((n, sequence_stride), poison, dtype=torch.int16, device="cuda")
    kvx.attend_prefill_batch(tw.dev, 1, QH, dq, together, tables, params, sequence_stride, ws)
    alone = torch.full((n, sequence_stride), poison, dtype=torch.int16, device="cuda")
    for i in range(n):
        kvx.attend_prefill(tw.dev, 1, QH, dq[i], alone[i], tables[i], params[i], ws)
    torch.cuda.synchronize()
    return Gp.host_u16(together), Gp.host_u16(alone), tw


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("committed,rows,planned", [
    ((1024, 2048, 512), 264, False),   # one split: paired (int4) or grouped lanes and an odd last tile
    ((1024, 2048, 512), 136, True),    # several splits by kvx_prefill_plan
    ((0, 4096), 2048, False),          # whole chunks, as the bench's prefill step has them
    ((1500, 2524, 476), 130, False),   # starts 4 tokens before a page boundary, rows not a multiple of 8
])
def test_equal_chunks_share_their_launches(fmt, committed, rows, planned):
    splits = kvx.lib().kvx_prefill_splits(rows)
    if planned:
        # one count for the batch: the smallest of the sequences' own plans
        splits = min(kvx.prefill_plan(c, rows, H, QH, fmt) for c in committed)
        assert splits > 1
    n = len(committed)
    before = kvx.attend_paths()
    together, alone, tw = run_batch(fmt, list(committed), [rows] * n, [splits] * n)
    after = kvx.attend_paths()
    assert after[0] == before[0], "head dimension 256 stays off the generic kernels"
    assert np.array_equal(together, alone)
    assert (alone != 0x5A5A).any()
    tw.close()


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8])
def test_more_sequences_than_one_launch_takes(fmt):
    """35 equal chunks: the launches take 32 sequences at a time, the last three their own."""
    n = 35
    committed = [32 * (1 + i % 3) for i in range(n)]
    splits = 2 if fmt == ko.INT8 else 1
    together, alone, tw = run_batch(fmt, committed, [72] * n, [splits] * n)
    assert np.array_equal(together, alone)
    assert (alone[-1] != 0x5A5A).any() and (alone[32] != 0x5A5A).any()
    tw.close()


@pytest.mark.parametrize("fmt", [ko.INT4, ko.BF16])
def test_unequal_chunks_run_one_after_the_other(fmt):
    committed, rows = [1000, 64, 3000], [77, 264, 8]
    splits = [int(kvx.lib().kvx_prefill_splits(r)) for r in rows]
    together, alone, tw = run_batch(fmt, committed, rows, splits)
    assert np.array_equal(together, alone)
    tw.close()


def test_one_invalid_sequence_enqueues_nothing():
    fmt = ko.INT4
    tw = Gp.Twin(fmt, H, D, 2, 8)
    pages, th, td = fill(tw, 128, seed=5)
    stride = 32
    q = Gp.dev(np.zeros((2, H * stride * G * D), dtype=np.uint16))
    out = torch.full((2, H * stride * G * D), 0x5A5A, dtype=torch.int16, device="cuda")
    ws = torch.empty(2 * kvx.prefill_workspace_bytes(tw.dev, 8, QH) + 256, dtype=torch.uint8, device="cuda")
    good = kvx.PrefillParams(64, 8, stride, len(pages), kvx.KvLayer(), 1, 0.0)
    short_table = kvx.PrefillParams(64, 8, stride, 1, kvx.KvLayer(), 1, 0.0)
    with pytest.raises(kvx.KvxError):
        kvx.attend_prefill_batch(tw.dev, 1, QH, q, out, [td, td], [good, short_table],
                                 H * stride * G * D, ws)
    with pytest.raises(kvx.KvxError):   # a sequence stride that overlaps the chunks
        kvx.attend_prefill_batch(tw.dev, 1, QH, q, out, [td, td], [good, good], 16, ws)
    torch.cuda.synchronize()
    assert (Gp.host_u16(out) == 0x5A5A).all()
    tw.close()
