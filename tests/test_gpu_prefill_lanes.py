"""Chunks of 64 rows and more on bf16, fp8 and int8 pages run in lanes of several 8-row tiles
whose four waves share every page through LDS; shorter chunks run a wave per tile or pair of
tiles.  Both walk the pages of a row in the same order with the same arithmetic, so a long
chunk in one call must give, bit for bit, the rows of the same chunk attended in pieces of
56 rows.  Verify lanes of more than 64 fused rows (bf16 pages: more than 32) run on the same kernels;
the layouts of tests/test_gpu_attention.py and tests/test_gpu_geometries.py give them 64, 96 and 128
rows, the most a verify lane may hold.  The pieces are the path that tests/test_gpu_attention.py holds against the
oracle.  Under several splits every split rounds its weights against its own running maximum,
so those results are held against the oracle with the same splits instead."""
import numpy as np
import pytest
import torch

from oracle import kvoracle as ko
from richengine_amd import kvx
import gpulib as Gp
import test_gpu_attention as A

pytestmark = pytest.mark.gpu
D = 256
WIDE = [ko.INT8, ko.BF16, ko.FP8]


def attend(tw, td, n_pages, heads, group, q, committed, rows, splits):
    stride = q.shape[1]
    out = torch.full((heads, stride, group, D), 0x5A5A, dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.prefill_workspace_bytes(tw.dev, rows, heads * group, splits), dtype=torch.uint8,
                     device="cuda")
    kvx.attend_prefill(tw.dev, 1, heads * group, Gp.dev(np.ascontiguousarray(q)), out, td,
                       kvx.PrefillParams(committed, rows, stride, n_pages, kvx.KvLayer(), splits, 0.0), ws)
    torch.cuda.synchronize()
    return Gp.host_u16(out)


@pytest.mark.parametrize("fmt,heads,group,committed,rows",
                         [(fmt, heads, group, committed, rows)
                          for fmt in WIDE for heads, group in [(4, 6), (4, 4), (2, 8)]
                          for committed, rows in [(0, 256), (1000, 296), (1024, 552)]] +
                         # groups at the ends of what the lanes of several tiles take: 3 query heads
                         # (96 fused rows in four tiles), 12 (192 in two), and 2, which they leave alone
                         [(fmt, heads, group, 1000, 296)
                          for fmt in (ko.INT8, ko.BF16) for heads, group in [(8, 3), (2, 12), (4, 2)]])
def test_long_chunk_is_its_short_pieces(fmt, heads, group, committed, rows):
    # 296 rows: 37 tiles, so lanes of four (or two) tiles and an odd tile on its own;
    # 1000 tokens before the chunk: its tiles start in the middle of a page
    tw = Gp.Twin(fmt, heads, D, 2, (committed + rows + 31) // 32)
    pages, th, td = A.fill(tw, committed + rows, seed=committed + rows + group)
    stride = (rows + 31) // 32 * 32
    q = np.zeros((heads, stride, group, D), dtype=np.uint16)
    q[:, :rows] = A.queries((heads, rows, group, D), committed + 5)
    before = kvx.attend_paths()
    whole = attend(tw, td, len(pages), heads, group, q, committed, rows, 1)
    for start in range(0, rows, 56):
        n = min(56, rows - start)
        piece_q = np.zeros((heads, 64, group, D), dtype=np.uint16)
        piece_q[:, :n] = q[:, start:start + n]
        piece = attend(tw, td, len(pages), heads, group, piece_q, committed + start, n, 1)
        assert np.array_equal(piece[:, :n], whole[:, start:start + n]), (start, n)
    assert not whole[:, rows:(rows + 7) // 8 * 8].any()
    assert (whole[:, (rows + 7) // 8 * 8:] == 0x5A5A).all()
    after = kvx.attend_paths()
    assert after[1] > before[1] and after[0] == before[0]
    tw.close()


@pytest.mark.parametrize("fmt,heads,group,committed,rows,splits",
                         [(fmt, *case) for fmt in (ko.INT8, ko.BF16)
                          for case in [(4, 6, 1024, 296, 3), (4, 4, 1024, 136, 3), (2, 8, 1024, 136, 3),
                                       (4, 6, 0, 256, 8), (4, 6, 1000, 264, 2)]] +
                         [(ko.FP8, 4, 6, 1024, 136, 3)])
def test_long_chunk_under_several_splits_matches_oracle(fmt, heads, group, committed, rows, splits):
    # after 1024 and 0 tokens the tiles of a lane cut their pages into the same splits and the
    # lanes of several tiles run; after 1000 they do not, and the chunk runs tile by tile
    saved = (A.H, A.G, A.QH)
    A.H, A.G, A.QH = heads, group, heads * group
    try:
        A.prefill_case(fmt, committed, rows, forced_splits=splits)
    finally:
        A.H, A.G, A.QH = saved

