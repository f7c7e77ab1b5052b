"""Calls from several host threads at once, each on a stream and a workspace of its own over one
storage: what a serving loop with a thread per request group does.  The library keeps no state
between calls except the pages, its error text is per thread, and its call counters are atomic,
so every thread must get the rows a lone caller gets, bit for bit."""
import threading

import numpy as np
import pytest
import torch

from oracle import kvoracle as ko
from richengine_amd import kvx
import gpulib as Gp
from test_gpu_attention import H, G, D, QH, queries, shared_pool_lanes

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fmt", [ko.INT4, ko.BF16])
def test_threads_on_their_own_streams_get_the_lone_callers_rows(fmt):
    committed = [0, 33, 700, 2047, 4095, 1500, 63, 3000]
    lanes = len(committed)
    tw, counts, hts, dts = shared_pool_lanes(fmt, committed, 1, seed=40 + fmt)
    splits = kvx.decode_plan(committed, H, fmt)
    dp = [kvx.VerifyParams(committed[i], counts[i], kvx.KvLayer(), splits[i], splits[i], 1, 1, 0.0)
          for i in range(lanes)]
    need = kvx.attend_workspace_bytes(tw.dev, dp, QH)
    threads, calls = 4, 40
    q = [Gp.dev(queries((lanes, H, 1, G, D), 70 + t)) for t in range(threads)]
    alone = []
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    for t in range(threads):
        out = torch.zeros((lanes, H, 1, G, D), dtype=torch.int16, device="cuda")
        kvx.attend_decode(tw.dev, 1, QH, q[t], out, dts, dp, 1, ws)
        torch.cuda.synchronize()
        alone.append(out.clone())
    before = kvx.attend_paths()
    failures = []

    def worker(t):
        try:
            stream = torch.cuda.Stream()
            space = torch.empty(need, dtype=torch.uint8, device="cuda")
            out = torch.zeros((lanes, H, 1, G, D), dtype=torch.int16, device="cuda")
            stream.wait_stream(torch.cuda.current_stream())
            for call in range(calls):
                kvx.attend_decode(tw.dev, 1, QH, q[t], out, dts, dp, 1, space, stream=stream.cuda_stream)
                if call % 8 == 7:   # an error on this thread keeps its text on this thread
                    with pytest.raises(kvx.KvxError) as e:
                        kvx.attend_decode(tw.dev, 99, QH, q[t], out, dts, dp, 1, space, stream=stream.cuda_stream)
                    assert "layer" in str(e.value).lower()
            stream.synchronize()
            if not torch.equal(out, alone[t]):
                failures.append((t, "rows differ from the lone caller's"))
        except Exception as e:   # reported by the main thread
            failures.append((t, repr(e)))

    workers = [threading.Thread(target=worker, args=(t,)) for t in range(threads)]
    for w in workers:
        w.start()
    for w in workers:
        w.join()
    torch.cuda.synchronize()
    assert not failures, failures
    after = kvx.attend_paths()
    assert sum(after) - sum(before) == threads * calls
    tw.close()
