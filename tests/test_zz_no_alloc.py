"""kv_attend_decode_static, the entry that allocates nothing: decode attention whose partial rows
and statistics go to the library's static device array instead of a caller's workspace.  Its
output must be kv_attend_decode's, bit for bit (the same kernels over other scratch memory), on
two calls in a row, the second with a smaller batch, and sizes past the array are refused with
nothing enqueued."""
import gc

import numpy as np
import pytest
import torch

from oracle import kvoracle as ko
from richengine_amd import kvx
import gpulib as Gp
import test_gpu_attention as A

pytestmark = pytest.mark.gpu
H, G, D = 4, 6, 256
QH = H * G


def test_static_workspace_decode_is_the_workspace_decode():
    committed = [0, 31, 700, 4095, 2047, 5000, 9000, 63]
    tw, counts, hts, dts = A.shared_pool_lanes(ko.INT4, committed, 1, seed=401)
    lanes = len(committed)
    q = Gp.dev(A.queries((lanes, H, 1, G, D), 402))
    splits = [max(kvx.lib().kvx_decode_splits(c, 1), 1 + (c > 600)) for c in committed]
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], splits[i], 1, 1, 0.0)
          for i in range(lanes)]
    ws = torch.empty(kvx.attend_workspace_bytes(tw.dev, dp, QH), dtype=torch.uint8, device="cuda")

    def both(first, count):
        want = torch.full((count, H, 1, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
        kvx.attend_decode(tw.dev, 1, QH, q[first:first + count], want, dts[first:first + count],
                          dp[first:first + count], 1, ws)
        got = torch.full_like(want, 0x5A5A)
        torch.cuda.synchronize()
        # Tensors that earlier tests left in reference cycles must not be released between the
        # two readings; free device memory as the driver reports it also sees an allocation that
        # does not go through torch.
        gc.collect()
        allocated, free = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        kvx.attend_decode_static(tw.dev, 1, QH, q[first:first + count], got, dts[first:first + count],
                                 dp[first:first + count], 1)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == allocated
        assert torch.cuda.mem_get_info()[0] == free
        assert torch.equal(got, want)
        return got

    whole = both(0, lanes)
    # against the oracle too, for one lane with several splits
    lane = 3
    q1 = np.zeros((1, H, 32, G, D), dtype=np.uint16)
    q1[0, :, 0] = Gp.host_u16(q)[lane, :, 0]
    hp = ko.VerifyParams(committed[lane], counts[lane], tw.host.layer(1), splits[lane], 128, 1, 1, 0.0)
    n, bits, f32 = ko.attend_verify(ko.INT4, H, G, D, q1, [hts[lane]], [hp])
    assert n == 1
    Gp.check_attention(Gp.host_u16(whole)[lane, :, 0], bits[0, :, 0], f32[0, :, 0],
                       np.ones(H, dtype=bool), 2e-3, "static workspace decode",
                       explain=lambda index: dict(fmt=ko.INT4, kv_heads=H, group=G, head_dim=D,
                                                  tile_queries=q1[0, index[0], 0], table=hts[lane],
                                                  kv=tw.host.layer(1), head=index[0],
                                                  committed=committed[lane], active=1,
                                                  splits=splits[lane], capacity=1, fused_row=index[1]))
    # the second call in a row is smaller: what the first left in the array must not show
    both(2, 3)
    both(5, 1)
    # under stream capture: the address of the array was looked up when the storage was made,
    # so the call records kernel launches only; every replay, with eager work and
    # synchronisations of the program's own between them, gives the eager rows
    assert kvx.lib().kvx_static_workspace_prime(tw.dev.h) == 0
    eager = torch.full((lanes, H, 1, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    kvx.attend_decode_static(tw.dev, 1, QH, q, eager, dts, dp, 1)
    torch.cuda.synchronize()
    assert torch.equal(eager, whole)
    captured = torch.full_like(eager, 0x5A5A)
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            kvx.attend_decode_static(tw.dev, 1, QH, q, captured, dts, dp, 1,
                                     stream=torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    for replay in range(3):
        captured.fill_(0x5A5A)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(captured, whole), f"replay {replay} of the captured call differs"
        both(replay, 2)                      # eager calls over the same array in between
    del graph
    # more partial rows than the array holds: refused, nothing enqueued
    huge = [kvx.VerifyParams(committed[3], counts[3], kvx.KvLayer(), 512, 512, 1, 1, 0.0)] * 32
    assert kvx.attend_workspace_bytes(tw.dev, huge, QH) > 32 << 20      # KVX_STATIC_WORKSPACE_BYTES
    out = torch.full((32, H, 1, G, D), 0x5A5A, dtype=torch.int16, device="cuda")
    q32 = q[:1].expand(32, H, 1, G, D).contiguous()
    with pytest.raises(kvx.KvxError) as refused:
        kvx.attend_decode_static(tw.dev, 1, QH, q32, out, [dts[3]] * 32, huge, 1)
    assert refused.value.code == kvx.EINVAL and "static workspace" in str(refused.value)
    torch.cuda.synchronize()
    assert (out == 0x5A5A).all()
    tw.close()
