"""How far the scores of the matrix-core kernels lie from the oracle's, measured.

The attention checks allow a row above the tolerance only when the oracle, with the rounding
of one or two heavy probabilities turned, lands on the GPU's row, and a rounding may only be
turned where the unrounded weight lies within a slack of a rounding boundary
(oracle/kvoracle.py: flip_slack).  That slack stands for the score deviation between the two
sides: a score that is off by d moves its probability by d, relatively.  The deviation can be
read off directly: every split reports the maximum of its scores and the sum of its
probabilities (kv_attend_split's statistics), and so does the oracle's tile.  The difference
of the maxima is the score deviation at the split's heaviest token; the difference of
max + log(sum) is the average deviation over the split's heavy tokens.

Per format, over long histories with 20x outlier channels in keys and queries, one-row
decode, 8-row chains and lanes of 12 and 16 rows, the worst deviation must stay under half of the slack that format
uses, and the measured figures go into the run's summary."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import kvoracle as ko
from richengine_amd import kvx
import gpulib as Gp
import kvtestlib as T

pytestmark = pytest.mark.gpu
H, G, D = 4, 6, 256
QH = H * G


def history(tw, layer, th, td, pages, tokens, seed):
    """Random rows with 20x outlier channels through kv_append; the oracle store gets the bytes."""
    gen = torch.Generator(device="cuda").manual_seed(seed)
    done = 0
    while done < tokens:
        n = min(2048, tokens - done)
        stride = (n + 31) // 32 * 32
        k = torch.randn((H, stride, D), generator=gen, device="cuda")
        v = torch.randn((H, D, stride), generator=gen, device="cuda")
        k[:, :, [3, 77, 130, 255]] *= 20
        v[:, [5, 64, 131, 250], :] *= 20
        kvx.append(tw.dev, layer, k.bfloat16(), v.bfloat16(), [td],
                   [kvx.ChunkParams(done, n, stride, pages)], H * stride * D)
        done += n


def oracle_statistics(fmt, tile_queries, table, kv, head, committed, active, splits, capacity):
    L = ko.lib()
    M = capacity * G
    partials = np.zeros((splits, M, D), dtype=np.float32)
    statistics = np.zeros((splits, M, 2), dtype=np.float32)
    q = np.ascontiguousarray(tile_queries, dtype=np.uint16).reshape(M, D)
    for split in range(splits):
        L.ko_attention_tile(fmt, H, G, D, capacity, ko.ptr(q), ko.ptr(table), kv, head, committed,
                            active, splits, split, ko.ptr(partials), ko.ptr(statistics), split, None,
                            0.0)
    return statistics


@pytest.mark.parametrize("query_outliers", [False, True])
@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16, ko.FP8])
def test_score_deviation_is_within_half_the_flip_slack(fmt, query_outliers):
    cases = [  # (committed, rows, splits); 16 rows are 96 fused rows: the kernels of wide lanes
        (20000, 1, 20), (8191, 1, 8), (4097, 8, 32), (12000, 8, 12), (6000, 16, 12), (147, 12, 9)]
    worst_max = worst_lse = 0.0
    samples = 0
    for number, (committed, rows, splits) in enumerate(cases):
        pages = (committed + rows + 31) // 32
        tw = Gp.Twin(fmt, H, D, 1, pages)
        th, td = tw.tables(tw.pages(pages, 500 + number))
        history(tw, 0, th, td, pages, committed + rows, 600 + number)
        torch.cuda.synchronize()
        tw.download()
        rng = np.random.default_rng(700 + number)
        qf = rng.standard_normal((1, H, rows, G, D)).astype(np.float32)
        if query_outliers:
            qf[..., [3, 77, 130, 255]] *= 20      # the query's outliers meet the keys'
        capacity = 1 if rows == 1 else 8 if rows <= 8 else 16
        q = np.zeros((1, H, 32 if rows > 1 else 1, G, D), dtype=np.uint16)
        q[:, :, :rows] = ko.f32_to_bf16(qf).reshape(1, H, rows, G, D)
        lane = kvx.VerifyParams(committed, pages, kvx.KvLayer(), splits, splits, rows, capacity, 0.0)
        M = capacity * G
        total_rows = splits * H * M
        statistics_at = (total_rows * D * 4 + 255) // 256 * 256
        ws = torch.zeros(statistics_at + total_rows * 8 + 256, dtype=torch.uint8, device="cuda")
        kvx.attend_split(tw.dev, 0, QH, Gp.dev(q), [td], [lane], None, q.shape[2], ws)
        torch.cuda.synchronize()
        got = ws[statistics_at:statistics_at + total_rows * 8].cpu().numpy().view(np.float32)
        got = got.reshape(H, splits, M, 2)
        for head in range(H):
            want = oracle_statistics(fmt, q[0, head, :capacity], th, tw.host.layer(0), head, committed,
                                     rows, splits, capacity)
            live = np.isfinite(want[..., 0]) & (want[..., 1] > 0)
            assert live.any() and np.array_equal(live, np.isfinite(got[head][..., 0]) & (got[head][..., 1] > 0))
            d_max = np.abs(got[head][..., 0][live].astype(np.float64) - want[..., 0][live])
            lse_got = got[head][..., 0][live].astype(np.float64) + np.log(got[head][..., 1][live].astype(np.float64))
            lse_want = want[..., 0][live].astype(np.float64) + np.log(want[..., 1][live].astype(np.float64))
            worst_max = max(worst_max, float(d_max.max()))
            worst_lse = max(worst_lse, float(np.abs(lse_got - lse_want).max()))
            samples += int(live.sum())
        tw.close()
    slack = ko.flip_slack(fmt)
    Gp.DEVIATION_LOG.append((ko.FORMAT_NAMES[fmt] + (", queries with the keys' outlier channels" if query_outliers else ""),
                             samples, worst_max, worst_lse, slack))
    assert worst_max <= slack / 2, (f"format {fmt}: a split's maximum score lies {worst_max:.2e} from the "
                                    f"oracle's, more than half of the flip slack {slack:.2e}")
    assert worst_lse <= slack / 2, (f"format {fmt}: max + log(sum) lies {worst_lse:.2e} from the oracle's, "
                                    f"more than half of the flip slack {slack:.2e}")
