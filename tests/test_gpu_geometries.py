"""The reference's other shipped layouts of head dimension 256 on the matrix-core kernels:
_kv4_g4 (4 KV heads x group 4) and _kv2_g8 (2 x 8) next to the default (4 x 6)
(runtime/ops/PagedAttention.cpp:66-115).  Groups of 4 and 8 give 4 / 32 / 64 and 8 / 64 / 128
fused rows for decode / chain verify / tree verify: other block counts, other rows past the
tile in the last block, other verify block choices (48-row waves at 33..48 and 65..96 fused
rows only) and other prefill pairing thresholds than the default layout's 6 / 48 / 96.
The cases are those of tests/test_gpu_attention.py, run with the layout switched."""
import numpy as np
import pytest

from oracle import kvoracle as ko
from richengine_amd import kvx
import test_gpu_attention as A

pytestmark = pytest.mark.gpu
LAYOUTS = {"kv4_g4": (4, 4), "kv2_g8": (2, 8)}


@pytest.fixture(params=sorted(LAYOUTS))
def layout(request):
    saved = (A.H, A.G, A.QH)
    A.H, A.G = LAYOUTS[request.param]
    A.QH = A.H * A.G
    before = kvx.attend_paths()
    yield request.param
    after = kvx.attend_paths()
    A.H, A.G, A.QH = saved
    # every call of these tests ran on the matrix-core kernels
    assert after[1] > before[1] and after[0] == before[0], (before, after)


@pytest.mark.parametrize("fmt", A.FORMATS)
def test_decode(layout, fmt):
    A.decode_case(fmt, [0, 31, 32, 511, 1000, 2047, 4095, 5000, 33], seed=180 + fmt)


@pytest.mark.parametrize("fmt", A.FORMATS)
def test_verify_chain(layout, fmt):
    A.test_verify_chain_matches_oracle(fmt)


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16])
def test_batched_verify_chain(layout, fmt):
    A.test_batched_verify_chain_matches_oracle(fmt)


@pytest.mark.parametrize("fmt", [ko.INT4, ko.INT8, ko.BF16])
@pytest.mark.parametrize("nodes", [15, 16])
def test_tree_verify(layout, fmt, nodes):
    A.test_tree_verify_matches_oracle(fmt, nodes)


@pytest.mark.parametrize("fmt", A.FORMATS)
@pytest.mark.parametrize("committed,rows", [(0, 1), (33, 7), (255, 17), (2000, 130), (1500, -136),
                                            (1508, -136)])
def test_prefill(layout, fmt, committed, rows):
    # rows < 0: kvx_prefill_plan's split count, where it gives this layout more than one
    if rows < 0 and kvx.prefill_plan(committed, -rows, A.H, A.QH, fmt) <= 1:
        rows = -rows
    A.prefill_case(fmt, committed, rows)


def test_int4_prefill_pairs(layout):
    # enough tiles to pair under several splits, starting 4 tokens before a page boundary
    splits = kvx.prefill_plan(284, 512, A.H, A.QH, ko.INT4)
    assert 1 <= splits <= 32
    A.prefill_case(ko.INT4, 284, -512 if splits > 1 else 512)


def test_append_attend_decode(layout):
    A.test_append_attend_decode_is_the_two_calls(ko.INT4)
