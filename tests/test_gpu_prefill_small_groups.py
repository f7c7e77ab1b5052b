"""Chunked prefill at head dimensions 64 and 128 on a history that ends on a page boundary, where
the tiles that begin in the same 32 (or 16) rows of the chunk share a workgroup and a staged page
(prefill_group_small_kernel; kvx_debug_prefill_tiles_together tells when).  Every tile keeps its own
pages, splits and slots, so the chunk's rows must be, bit for bit, those of the same tiles run one by
one (a call of 8 rows per tile, which the tile-by-tile kernel serves), and they are held to the
oracle like any other prefill."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import kvoracle as ko
from richengine_amd import kvx
import gpulib as Gp
import test_gpu_attention as A

pytestmark = pytest.mark.gpu

# (KV heads, group, head dimension) -> tiles together in a large enough launch: 1 and 2 blocks of
# 16 fused rows to a tile at 128 (4 and 2 tiles), 1 .. 4 blocks at 64 (4, 4, 2, 2); more blocks
# stay tile by tile
LAYOUTS = {(4, 2, 128): 4, (2, 4, 128): 2, (3, 5, 128): 1, (2, 8, 128): 1, (4, 2, 64): 4, (8, 4, 64): 4,
           (4, 6, 64): 2, (2, 8, 64): 2, (2, 13, 64): 1}


def together(layout, fmt, committed, rows, splits):
    heads, group, dim = layout
    l = kvx.Layout(1, heads, dim, fmt, 0.0)
    return kvx.lib().kvx_debug_prefill_tiles_together(C.byref(l), heads * group, committed, rows, splits)


@pytest.fixture
def layout(request):
    saved = (A.H, A.G, A.D, A.QH)
    A.H, A.G, A.D = request.param
    A.QH = A.H * A.G
    yield request.param
    A.H, A.G, A.D, A.QH = saved


@pytest.mark.parametrize("layout", sorted(LAYOUTS), indirect=True)
@pytest.mark.parametrize("fmt", A.FORMATS)
def test_grouped_tiles_match_the_oracle(layout, fmt):
    rng = np.random.default_rng(sum(layout) + fmt)
    # a launch too small for groups, then one of the size that takes them: 32 splits of a ragged
    # chunk (the last group and the last tile partly filled)
    cases = ((0, 40, 1, False), (32 * int(rng.integers(4, 14)), 251, 32, True))
    heads, group, dim = layout
    planned = kvx.lib().kvx_prefill_plan_for(C.byref(kvx.Layout(1, heads, dim, fmt, 0.0)), 32 * 40, 251, heads * group, 1)
    assert 1 <= planned <= 12        # 48 pages: at least 4 to a split
    cases += ((32 * 40, 251, planned, None),)
    for committed, rows, splits, large in cases:
        if large is None:            # the plan's splits, grouped or not as the rule has it
            A.prefill_case(fmt, committed, rows, forced_splits=splits)
            continue
        print(f"grouped prefill layout={layout} fmt={fmt} committed={committed} rows={rows} splits={splits}",
              flush=True)
        assert together(layout, fmt, committed, rows, splits) == (LAYOUTS[layout] if large else 1)
        assert together(layout, fmt, committed + 1, rows, splits) == 1
        A.prefill_case(fmt, committed, rows, forced_splits=splits)


@pytest.mark.parametrize("layout", sorted(LAYOUTS), indirect=True)
@pytest.mark.parametrize("fmt", [ko.INT4, ko.BF16])
def test_grouped_tiles_have_the_bits_of_tiles_run_alone(layout, fmt):
    H, G, D = layout
    QH = H * G
    committed, rows, splits = 32 * 11, 253, 32
    assert together(layout, fmt, committed, rows, splits) == LAYOUTS[layout]
    tw = Gp.Twin(fmt, H, D, 2, (committed + rows + 31) // 32)
    pages, th, td = A.fill(tw, committed + rows, seed=5)
    stride = 256
    q = np.zeros((H, stride, G, D), dtype=np.uint16)
    q[:, :rows] = A.queries((H, rows, G, D), 7)
    out = torch.zeros((H, stride, G, D), dtype=torch.int16, device="cuda")
    ws = torch.empty(kvx.prefill_workspace_bytes(tw.dev, rows, QH, splits), dtype=torch.uint8, device="cuda")
    kvx.attend_prefill(tw.dev, 1, QH, Gp.dev(q), out, td,
                       kvx.PrefillParams(committed, rows, stride, len(pages), kvx.KvLayer(), splits, 0.0), ws)
    torch.cuda.synchronize()
    grouped = Gp.host_u16(out)
    # tile k alone: its 8 rows as a chunk of their own behind committed + 8 k tokens
    one = torch.zeros((H, 32, G, D), dtype=torch.int16, device="cuda")
    for k in range((rows + 7) // 8):
        n = min(8, rows - 8 * k)
        q1 = np.zeros((H, 32, G, D), dtype=np.uint16)
        q1[:, :n] = q[:, 8 * k:8 * k + n]
        kvx.attend_prefill(tw.dev, 1, QH, Gp.dev(q1), one, td,
                           kvx.PrefillParams(committed + 8 * k, n, 32, len(pages), kvx.KvLayer(), splits, 0.0), ws)
        torch.cuda.synchronize()
        assert np.array_equal(Gp.host_u16(one)[:, :n], grouped[:, 8 * k:8 * k + n]), (layout, fmt, k)
    tw.close()
