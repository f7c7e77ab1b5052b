#!/usr/bin/env python3
"""Benchmark of the paged-KV decode path on one MI355X.

Workload (the configuration the headline metric is quoted on): int4 KV,
16 layers, 4 KV heads x 256, 24 query heads, batch 32 with contexts drawn
uniformly from [512, 32768]; pages come from a device-sized pool in a
seed-shuffled order, reached through per-sequence page tables.  One step is one
decode step of the whole batch: per layer, append one token per sequence
(quantize + scatter) and run paged decode attention (split partials + merge),
through kv_append_attend_decode (or the two separate entries with
--separate-append).

Prints ONE JSON line: whole-step KV GB/s (algorithmic KV bytes read by attention
/ step time), decode tokens/s, the roofline of the dominant kernel measured
with events on the launch stream, and the CPU oracle timed on a bounded sample.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# Kernel arguments in device memory rather than in host memory (HIP reads this when
# its runtime starts, which is after this line): every wave of the attention
# kernels finds its sequence in a 1.9 KB argument block, and fetching that from
# the host costs the merge kernel 2 us and a decode step 3 % (1.96 -> 1.89 ms).
# A caller's own setting wins.
os.environ.setdefault("HIP_FORCE_DEV_KERNARG", "1")

HBM_PEAK_GBS = 8000.0
H, G, D, LAYERS = 4, 6, 256, 16
QH = H * G
BATCH = 32
BYTES_PER_TOKEN_LAYER = 1056  # int4: 2 * (4 heads * 128 B + 4 * 4 B scales)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--seed", type=int, default=20261126,
                    help="the default draw of 32 contexts totals 535 067 tokens, 0.5%% above the mean "
                         "of U[512,32768] x 32 (532 480)")
    ap.add_argument("--pool-gb", type=float, default=0.0,
                    help="KV pool size; 0 = 80%% of free HBM, at most 256 GB")
    ap.add_argument("--contiguous", action="store_true",
                    help="hand out pages in order instead of shuffled (TLB comparison)")
    ap.add_argument("--cpu-seconds", type=float, default=30.0,
                    help="CPU oracle budget; 0 skips the CPU baseline")
    ap.add_argument("--kernel-iters", type=int, default=20)
    ap.add_argument("--uniform-context", type=int, default=0,
                    help="give every sequence this context instead of U[512,32768] (experiments)")
    ap.add_argument("--copy-calibration-pages", type=int, default=0,
                    help="before the timed region copy this many pool pages once with "
                         "kv_page_copy: a plain copy of known size to scale HBM counters by")
    ap.add_argument("--pages-per-split", type=int, default=0,
                    help="override the library's decode split rule (experiments)")
    ap.add_argument("--separate-append", action="store_true",
                    help="call kv_append and kv_attend_decode instead of kv_append_attend_decode")
    ap.add_argument("--hidden", choices=["none", "gate", "gather"], default="none",
                    help="decode: the merge also writes the out-projection's operand "
                         "(kv_append_attend_decode_hidden; with --separate-append kv_append + "
                         "kv_attend_verify_hidden), gated by packed projection rows or plainly gathered")
    ap.add_argument("--prepare", action="store_true",
                    help="decode: the step's queries, keys and values come from packed projection rows "
                         "through kv_prepare_append (norm, rotation, quantize, store) instead of "
                         "ready chunk rows through kv_append; implies --separate-append")
    ap.add_argument("--prefill-chunk", type=int, default=2048, choices=[64, 128, 256, 512, 1024, 2048],
                    help="prefill: rows per chunk (BASELINE configs[3] has 2048); smaller chunks show "
                         "what kvx_prefill_plan's split counts do")
    ap.add_argument("--prefill-streams", type=int, default=None,
                    help="prefill: HIP streams the batch's sequences are spread over (1 = all on the "
                         "current stream); a sequence's layers stay in order on its stream.  0 = the "
                         "batch in one kv_attend_prefill_batch call per layer on one stream.  Default: "
                         "0 on int4 pages, 4 otherwise (the faster of the two by a few per cent)")
    ap.add_argument("--verify-splits", type=int, default=0,
                    help="tree-verify: splits per sequence instead of the library's plan (experiments)")
    ap.add_argument("--workload", choices=["decode", "decode-single", "tree-verify", "prefill", "qkv-prepare", "shared-prefix",
                                           "stream-ceiling", "control-plane", "decode-layout", "prefill-layout"], default="decode",
                    help="decode = batch-32 mixed-length int4 decode, the headline metric (default); "
                         "decode-single = one sequence of 32768 tokens, the 16 per-layer calls replayed "
                         "as one HIP graph; tree-verify = 16-node tree verify and prefill = chunked prefill with a shared "
                         "prefix, the matrix-core paths (profiling); stream-ceiling = what the memory system "
                         "delivers for the headline batch's bytes under request shapes other than the "
                         "decode kernel's (linear, 16-byte coalesced, page order, pool size); control-plane = "
                         "the host calls of a batch-32 step (prefix page cache, sequence records), no GPU work; "
                         "decode-layout = one-row decode, prefill-layout = a prefill chunk, over the reference's "
                         "other layouts (--layout)")
    ap.add_argument("--layout", choices=["hd128", "hd64", "k2q4d128", "k4q2d128"], default="hd128",
                    help="decode-layout, prefill-layout: 2 KV heads x 8 x 128 or 8 x 4 x 64; prefill-layout "
                         "also 2 x 4 x 128 and 4 x 2 x 128")
    ap.add_argument("--format", choices=["bf16", "fp8", "int8", "int4"], default=None,
                    help="page format of the prefill workload (default bf16) and of the shared-prefix "
                         "and tree-verify workloads (default int4; no fp8)")
    args = ap.parse_args()
    if args.format is None:
        args.format = "int4" if args.workload in ("shared-prefix", "tree-verify", "decode-layout",
                                                   "prefill-layout") else "bf16"
    return args


def host_cpus():
    """What the CPU figures ran on: the machine's processors, those this process may use, and
    the threads the all-core legs start at most (a one-GPU box's share of its host)."""
    return {"host_cpus": os.cpu_count(), "affinity_cpus": len(os.sched_getaffinity(0)),
            "threads_cap": 16}


def cpu_lane_prepare(ctx, seed, H=H, G=G, D=D, fmt=None):
    """One sequence on the oracle: fills the history (untimed) and returns run(), the decode
    step of one layer (append one token, attend), which returns its seconds."""
    import numpy as np
    from oracle import kvoracle as ko

    page_format = ko.INT4 if fmt is None else fmt
    rng = np.random.default_rng(seed)
    n_pages = (ctx + 1 + 31) // 32
    store = ko.Store(1, H, D, page_format, n_pages, n_pages)
    store.allocate(0)
    table = store.entries(np.arange(n_pages, dtype=np.uint32))
    done = 0
    while done < ctx:
        n = min(2048, ctx - done)
        stride = (n + 31) // 32 * 32
        k = ko.f32_to_bf16(rng.standard_normal((H, stride, D)).astype(np.float32)).reshape(H, stride, D)
        v = ko.f32_to_bf16(rng.standard_normal((H, D, stride)).astype(np.float32)).reshape(H, D, stride)
        ko.store_chunk(page_format, H, D, k, v, table, ko.ChunkParams(done, n, stride, n_pages, store.layer(0)))
        done += n
    k = ko.f32_to_bf16(rng.standard_normal((H, 32, D)).astype(np.float32)).reshape(H, 32, D)
    v = ko.f32_to_bf16(rng.standard_normal((H, D, 32)).astype(np.float32)).reshape(H, D, 32)
    q = np.zeros((1, H, 32, G, D), dtype=np.uint16)
    q[0, :, 0] = ko.f32_to_bf16(rng.standard_normal((H, G, D)).astype(np.float32)).reshape(H, G, D)
    splits = min(max(1, ((ctx + 1 + 31) // 32 + 31) // 32), 128)

    def run():
        t0 = time.perf_counter()
        ko.store_chunk(page_format, H, D, k, v, table, ko.ChunkParams(ctx, 1, 32, n_pages, store.layer(0)))
        ko.attend_verify(page_format, H, G, D, q, [table],
                         [ko.VerifyParams(ctx, n_pages, store.layer(0), splits, 128, 1, 1, 0.0)],
                         want_f32=False)
        return time.perf_counter() - t0

    run.close = store.close
    return run


def cpu_lane(ctx, seed, **layout):
    """History filled untimed, then the timed decode step of one layer.  Returns seconds."""
    run = cpu_lane_prepare(ctx, seed, **layout)
    spent = run()
    run.close()
    return spent


def cpu_baseline(contexts, seed, budget_s):
    """The oracle (scalar C++ port) on a bounded sample of the same workload: whole sequences
    of the batch, shortest first, one layer each (append one token, then decode attention).
    First on one thread; then the same sequences on the host's cores, one sequence per thread
    (the oracle's calls release the interpreter lock), all histories filled first and the
    decode steps started together, timed by the wall clock from the common start to the last
    thread's end.  One layer of the whole batch would take the sample's time times
    `layer_over_sample`: the work is linear in the tokens."""
    import concurrent.futures
    import threading
    import numpy as np

    order = [int(i) for i in np.argsort(contexts)]  # shortest first so the sample stays bounded
    spent, sample = 0.0, []
    for lane in order:
        ctx = int(contexts[lane])
        tokens = sum(int(contexts[i]) + 1 for i in sample)
        if spent > 0 and spent + spent / max(tokens, 1) * ctx > 0.8 * budget_s:
            break
        spent += cpu_lane(ctx, seed + lane)
        sample.append(lane)
    tokens = sum(int(contexts[i]) + 1 for i in sample)
    nbytes = tokens * BYTES_PER_TOKEN_LAYER
    layer_tokens = sum(int(c) + 1 for c in contexts)
    host = host_cpus()
    cores = max(1, min(host["threads_cap"], host["affinity_cpus"], len(sample)))
    # longest first, so that the threads' shares come out even
    runs = [cpu_lane_prepare(int(contexts[lane]), seed + lane) for lane in sample[::-1]]
    start = threading.Barrier(cores + 1)
    queue, lock = list(runs), threading.Lock()

    def worker():
        start.wait()
        while True:
            with lock:
                if not queue:
                    return
                run = queue.pop(0)
            run()

    with concurrent.futures.ThreadPoolExecutor(cores) as pool:
        futures = [pool.submit(worker) for _ in range(cores)]
        start.wait()
        t0 = time.perf_counter()
        for f in futures:
            f.result()
        wall = time.perf_counter() - t0
    for run in runs:
        run.close()
    return {
        "value": nbytes / spent / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": f"{len(sample)} shortest sequences of the batch of {len(contexts)} ({tokens} of the "
                  f"layer's {layer_tokens} tokens), one layer: append 1 token + decode attention each, "
                  f"{spent:.1f} s of scalar C++ oracle",
        "layer_over_sample": round(layer_tokens / tokens, 2),
        "one_layer_of_the_batch_s": round(spent * layer_tokens / tokens, 1),
        "decode_tokens_per_s_one_layer": len(sample) / spent,
        **host,
        "all_cores": {"cores": cores, "value": nbytes / wall / 1e9, "unit": "GB/s",
                      "wall_s": round(wall, 2),
                      "one_layer_of_the_batch_s": round(wall * layer_tokens / tokens, 1),
                      "note": "same sequences over the threads, longest first; wall clock from the "
                              "threads' common start to the last one's end, history fills before it"},
    }


def cpu_history(ko, rng, fmt, tokens):
    """An oracle store of one layer holding `tokens` tokens of N(0,1) rows (untimed fill);
    returns (store, table, pages)."""
    import numpy as np
    n_pages = (tokens + 31) // 32 + 1
    store = ko.Store(1, H, D, fmt, n_pages, n_pages)
    store.allocate(0)
    table = store.entries(np.arange(n_pages, dtype=np.uint32))
    done = 0
    while done < tokens:
        n = min(2048, tokens - done)
        stride = (n + 31) // 32 * 32
        k = ko.f32_to_bf16(rng.standard_normal((H, stride, D)).astype(np.float32)).reshape(H, stride, D)
        v = ko.f32_to_bf16(rng.standard_normal((H, D, stride)).astype(np.float32)).reshape(H, D, stride)
        ko.store_chunk(fmt, H, D, k, v, table, ko.ChunkParams(done, n, stride, n_pages, store.layer(0)))
        done += n
    return store, table, n_pages


def cpu_tree_verify(seed, context, nodes, masks, budget_s):
    """The oracle on a bounded sample of the tree-verify workload: one sequence, one layer,
    the append of the tree's rows and the masked verify over a history cut to what the budget
    allows (cost is linear in the history); the rate is scaled back to the full history and to
    16 layers."""
    import numpy as np
    from oracle import kvoracle as ko
    rng = np.random.default_rng(seed)
    # ~1 GFLOP/s for the scalar port: rows x heads x D x 4 flops per visible token
    per_token = 4.0 * D * nodes * QH / 1.0e9
    history = int(min(context, max(2048, (budget_s / per_token) // 2048 * 2048)))
    store, table, n_pages = cpu_history(ko, rng, ko.INT4, history)
    k = ko.f32_to_bf16(rng.standard_normal((H, 32, D)).astype(np.float32)).reshape(H, 32, D)
    v = ko.f32_to_bf16(rng.standard_normal((H, D, 32)).astype(np.float32)).reshape(H, D, 32)
    q = ko.f32_to_bf16(rng.standard_normal((1, H, 32, G, D)).astype(np.float32)).reshape(1, H, 32, G, D)
    splits = min(max(1, n_pages // 64), 128)
    t0 = time.perf_counter()
    stored = ko.store_verify(ko.INT4, H, D, k[None], v[None], [table],
                             [ko.ChunkParams(history, nodes, 32, n_pages, store.layer(0))], 16)
    attended = ko.attend_verify(ko.INT4, H, G, D, q, [table],
                                [ko.VerifyParams(history, n_pages, store.layer(0), splits, 128, nodes, 16,
                                                 0.0)],
                                row_masks=np.ascontiguousarray(masks[:1]), want_f32=False)[0]
    spent = time.perf_counter() - t0
    store.close()
    assert stored == 1 and attended == 1, "the oracle refused the tree-verify sample"
    full = spent * (context + nodes) / (history + nodes) * LAYERS  # one sequence, all layers, full history
    return {"value": nodes / full, "unit": "draft tokens/s", "cores": 1, "kind": "port", **host_cpus(),
            "sample": f"one sequence of the batch, one layer, history cut to {history} of {context} tokens: "
                      f"append {nodes} tree rows + masked verify, {spent:.1f} s of scalar C++ oracle; "
                      f"scaled linearly to the full history and {LAYERS} layers",
            "seconds": spent, "history_tokens": history}


def cpu_prefill(seed, fmt_name, prefix, chunk, budget_s):
    """The oracle on a bounded sample of the chunked-prefill workload: one sequence, one layer,
    the first rows of one chunk (append + causal attention over the prefix and those rows), as
    many rows as the budget allows; the rate is per 16 layers."""
    import numpy as np
    from oracle import kvoracle as ko
    fmt = {"bf16": ko.BF16, "fp8": ko.FP8, "int8": ko.INT8, "int4": ko.INT4}[fmt_name]
    rng = np.random.default_rng(seed)
    per_row = 4.0 * D * QH * prefix / 1.0e9  # seconds per chunk row at ~1 GFLOP/s
    rows = int(min(chunk, max(8, (budget_s / per_row) // 8 * 8)))
    store, table, n_pages = cpu_history(ko, rng, fmt, prefix + rows)
    # cpu_history filled prefix + rows tokens; the chunk's rows are stored again by the timed append
    stride = (rows + 31) // 32 * 32
    k = ko.f32_to_bf16(rng.standard_normal((H, stride, D)).astype(np.float32)).reshape(H, stride, D)
    v = ko.f32_to_bf16(rng.standard_normal((H, D, stride)).astype(np.float32)).reshape(H, D, stride)
    q = ko.f32_to_bf16(rng.standard_normal((H, stride, G, D)).astype(np.float32)).reshape(H, stride, G, D)
    t0 = time.perf_counter()
    stored = ko.store_chunk(fmt, H, D, k, v, table,
                            ko.ChunkParams(prefix, rows, stride, n_pages, store.layer(0)))
    attended = ko.attend_prefill(fmt, H, G, D, q, table,
                                 ko.PrefillParams(prefix, rows, stride, n_pages, store.layer(0), 1, 0.0),
                                 want_f32=False)[0]
    spent = time.perf_counter() - t0
    store.close()
    assert stored == 1 and attended == 1, "the oracle refused the prefill sample"
    return {"value": rows / (spent * LAYERS), "unit": "tokens/s", "cores": 1, "kind": "port", **host_cpus(),
            "sample": f"one sequence, one layer, the first {rows} rows of a {chunk}-row chunk over the "
                      f"{prefix}-token prefix: append + causal attention, {spent:.1f} s of scalar C++ "
                      f"oracle; rate = rows / (seconds x {LAYERS} layers)",
            "seconds": spent, "rows": rows}



def cpu_qkv_prepare(seed, budget_s):
    """The oracle on the qkv-prepare workload's chunk, one layer: 2048 rows prepared (norm,
    rotation, layout) and stored into int4 pages."""
    import numpy as np
    from oracle import kvoracle as ko
    rng = np.random.default_rng(seed)
    pairs, width = 32, (2 * QH + 2 * H) * D
    rows = 2048                                                      # the whole chunk: a fraction of a second
    n_pages = rows // 32 + 1
    store = ko.Store(1, H, D, ko.INT4, n_pages, n_pages)
    store.allocate(0)
    table = store.entries(np.arange(n_pages, dtype=np.uint32))
    bf = lambda a: ko.f32_to_bf16(a.astype(np.float32)).reshape(a.shape)
    packed = bf(rng.standard_normal((rows, width)))
    wq, wk = bf(rng.standard_normal(D)), bf(rng.standard_normal(D))
    cos = rng.random((rows, pairs), dtype=np.float32)
    sin = rng.random((rows, pairs), dtype=np.float32)
    t0 = time.perf_counter()
    _, k, v = ko.qkv_prepare(H, G, D, pairs, True, 1e-6, rows, rows, packed, wq, wk, cos, sin)
    stored = ko.store_chunk(ko.INT4, H, D, k, v, table, ko.ChunkParams(0, rows, rows, n_pages, store.layer(0)))
    spent = time.perf_counter() - t0
    store.close()
    assert stored == 1, "the oracle refused the qkv-prepare sample"
    return {"value": rows / spent, "unit": "tokens/s", "cores": 1, "kind": "port", **host_cpus(),
            "sample": f"the whole {rows}-row chunk, one layer: prepare + quantize + store, "
                      f"{spent:.2f} s of scalar C++ oracle",
            "seconds": spent, "rows": rows}


def profiled_traffic():
    """HBM bytes per launch of the split kernel on this workload, from the
    committed counter summary (two rocprofv3 --pmc runs of this script, scaled by
    what the same counters read for the library's page-copy kernel); None when
    the summary is absent."""
    path = os.path.join(ROOT, "profiles", "decode_int4_batch32_hbm_traffic.txt")
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch:"):
                return int(float(line.split(":", 1)[1]))
    except OSError:
        pass
    return None


MFMA_BF16_PEAK_TFLOPS = 2500.0


def tree_verify(args):
    """Speculative tree verify: int4, batch 4, contexts 65536, a 16-node draft tree per
    sequence (branching <= 3).  A step = per layer, append the 16 draft rows and
    run masked verify attention over history + rows; then compact a seeded
    root-to-leaf path of every sequence, all layers in one call.  The dominant
    kernel (verify32_int4_kernel) runs on the matrix cores; its line carries the
    MFMA roofline (flops = 4 x D x fused query rows x visible tokens per layer)."""
    import numpy as np
    import torch
    from richengine_amd import kvx

    L = kvx.lib()
    torch.cuda.set_device(0)
    rng = np.random.default_rng(args.seed)
    lanes, context, nodes = 4, 65536, 16
    n_pages = (context + nodes + 31) // 32
    if args.format not in ("int4", "int8", "bf16"):
        sys.exit("tree verify runs on int4 (BASELINE configs[4]), int8 or bf16 pages")
    fmt = {"int4": kvx.INT4, "int8": kvx.INT8, "bf16": kvx.BF16}[args.format]
    bytes_per_token = {"int4": BYTES_PER_TOKEN_LAYER, "int8": 2080, "bf16": 4096}[args.format]
    layout = kvx.Layout(LAYERS, H, D, fmt, 0.0)
    extent_pages = L.kvx_layout_largest_extent_pages(C.byref(layout))
    extents = -(-lanes * n_pages // extent_pages)
    storage = kvx.Storage(LAYERS, H, D, fmt, extents * extent_pages, extent_pages, aligned=True)
    # The pages belong to the pool and reach the sequences through their records, as in an
    # engine: everything is acquired once and given back in a seed-shuffled order, so the
    # sequences' pages come off the free stacks scattered over the extents.
    pool = kvx.Pool(storage, storage.page_count)
    prefix_cache = kvx.Prefix(pool)
    sequences = kvx.Sequences(pool, prefix_cache)
    for page in rng.permutation(pool.acquire(min(storage.page_count, lanes * n_pages + 64))):
        pool.release(int(page))
    tables, revisions = [], []
    for lane in range(lanes):
        sequences.begin(lane + 1)
        sequences.ensure_tokens(lane + 1, context + nodes)
        view = sequences.view(lane + 1)
        tables.append(storage.table(np.array(view["pages"], dtype=np.uint32)))
        revisions.append(view["revision"])
    gen = torch.Generator(device="cuda")
    gen.manual_seed(args.seed)
    for lane in range(lanes):
        for done in range(0, context, 2048):
            k = torch.randn((H, 2048, D), generator=gen, device="cuda").bfloat16()
            v = torch.randn((H, D, 2048), generator=gen, device="cuda").bfloat16()
            for layer in range(LAYERS):
                kvx.append(storage, layer, k, v, [tables[lane]],
                           [kvx.ChunkParams(done, 2048, 2048, n_pages)], H * 2048 * D)
    none = 0xFFFFFFFF
    masks = np.zeros((lanes, nodes), dtype=np.uint32)
    paths = np.zeros((lanes, 16), dtype=np.uint32)
    counts = np.zeros(lanes, dtype=np.uint32)
    for lane in range(lanes):
        parents, children = [none], {}
        for row in range(1, nodes):
            parent = int(rng.choice([c for c in range(row) if children.get(c, 0) < 3][-4:]))
            children[parent] = children.get(parent, 0) + 1
            parents.append(parent)
        masks[lane] = kvx.tree_masks(parents)
        leaf = int(rng.choice([c for c in range(nodes) if c not in children]))
        walk = []
        while leaf != none:
            walk.append(leaf)
            leaf = parents[leaf]
        walk.reverse()
        assert kvx.tree_path_valid(parents, walk)
        paths[lane, :len(walk)], counts[lane] = walk, len(walk)
    masks_d = torch.from_numpy(masks.view(np.int32)).cuda()
    paths_d = torch.from_numpy(paths.view(np.int32)).cuda()
    counts_d = torch.from_numpy(counts.view(np.int32)).cuda()
    chunk_k = torch.randn((lanes, H, 32, D), generator=gen, device="cuda").bfloat16()
    chunk_v = torch.randn((lanes, H, D, 32), generator=gen, device="cuda").bfloat16()
    queries = torch.randn((lanes, H, 32, G, D), generator=gen, device="cuda").bfloat16()
    output = torch.zeros_like(queries)
    splits = args.verify_splits or kvx.verify_plan([context] * lanes, nodes, H, QH, fmt)[0]
    cp = [kvx.ChunkParams(context, nodes, 32, n_pages) for _ in range(lanes)]
    vp = [kvx.VerifyParams(context, n_pages, kvx.KvLayer(), splits, splits, nodes, 16, 0.0)
          for _ in range(lanes)]
    workspace = torch.empty(kvx.attend_workspace_bytes(storage, vp, QH) + 4096, dtype=torch.uint8,
                            device="cuda")
    torch.cuda.synchronize()

    released = [0]

    def step():
        for lane in range(lanes):
            # room for the step's draft rows; a page list that changed is written out again
            sequences.ensure_tokens(lane + 1, context + nodes)
            view = sequences.view(lane + 1)
            if view["revision"] != revisions[lane]:
                tables[lane] = storage.table(np.array(view["pages"], dtype=np.uint32))
                revisions[lane] = view["revision"]
        for layer in range(LAYERS):
            kvx.append(storage, layer, chunk_k, chunk_v, tables, cp, H * 32 * D, verify_max_rows=16)
            kvx.attend_verify(storage, layer, QH, queries, output, tables, vp, masks_d, 32, workspace)
        kvx.compact_path(storage, 0xFFFFFFFF, tables, cp, paths_d, counts_d, 16)
        for lane in range(lanes):
            # the rollback's host side: pages that hold rejected rows only go back to the pool
            # (none at this context, whose draft rows share a page with the accepted ones;
            # the history itself stays where it is, so every step sees the same lanes)
            released[0] += sequences.truncate(lane + 1, context + int(counts[lane]))
            revisions[lane] = sequences.view(lane + 1)["revision"] if released[0] else revisions[lane]

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    def time_split():
        # the split dispatch alone (kv_attend_split), events on the launch stream
        kvx.attend_split(storage, 0, QH, queries, tables, vp, masks_d, 32, workspace)
        torch.cuda.synchronize()
        k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        k0.record()
        for it in range(args.kernel_iters):
            kvx.attend_split(storage, it % LAYERS, QH, queries, tables, vp, masks_d, 32, workspace)
        k1.record()
        torch.cuda.synchronize()
        return k0.elapsed_time(k1) / args.kernel_iters

    kernel_ms = time_split()
    visible = lanes * (context + nodes)
    flops = 4 * D * (nodes * QH) * visible  # q.k and p.v, multiply and add, every row over every token
    kv_bytes = visible * bytes_per_token
    achieved = flops / (kernel_ms * 1e-3) / 1e12
    result = {
        "metric": args.format + " tree verify (16-node trees, batch 4 x 65536 tokens): verified draft tokens/s",
        "value": round(lanes * nodes * args.steps / wall, 1), "unit": "draft tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall * 1e3 / args.steps, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"int4": "int4 pages, bf16 MFMA", "int8": "int8 pages, fp16 MFMA",
                  "bf16": "bf16 pages, bf16 MFMA"}[args.format] + ", fp32 accumulate", "data": "synthetic",
        "config": {"workload": "BASELINE configs[4]: speculative tree verify on " + args.format + " KV, batch 4, "
                               "contexts 65536, 16-node trees (branching <= 3), 16 layers: append 16 "
                               "rows + masked verify per layer, then path compaction over all layers",
                   "batch": lanes, "layers": LAYERS, "format": args.format,
                   "splits_per_sequence": int(splits), "seed": args.seed,
                   "pages_released_by_rollbacks": released[0]},
        # Verify of 16 rows is a bandwidth-bound path by its bytes (each page is read once for
        # 96 fused rows); what holds the kernel is the work per page of its matrix and vector
        # units, so the MFMA figures stand beside the HBM ones.
        "roofline": {"bound": "hbm", "achieved": round(kv_bytes / (kernel_ms * 1e-3) / 1e9, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(kv_bytes / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": None, "bytes_per_launch": kv_bytes,
                     "mfma_tflops": round(achieved, 1), "mfma_peak_tflops": MFMA_BF16_PEAK_TFLOPS,
                     "mfma_frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4),
                     "kernel": ("verify32_int4_kernel (split kernel of verify attention, three waves of 32 fused rows)"
                                if args.format == "int4" else
                                "group_wide_kernel (split kernel of verify attention, four waves of 24 fused "
                                "rows that share every page through LDS)") + ", one layer per launch",
                     "flops_per_launch": flops, "ms_per_launch": round(kernel_ms, 4),
                     "kv_gbs": round(kv_bytes / (kernel_ms * 1e-3) / 1e9, 1)},
        "cpu_baseline": None,
    }
    for lane in range(lanes):
        sequences.end(lane + 1)
    sequences.close()
    prefix_cache.close()
    pool.close()
    storage.close()
    if args.cpu_seconds > 0 and args.format == "int4":
        result["cpu_baseline"] = cpu_tree_verify(args.seed, context, nodes, masks, args.cpu_seconds)
    print(json.dumps(result))


def stream_ceiling(args):
    """Where the distance between the decode kernel and the 8 TB/s peak lies: the bytes of one
    layer of the headline batch (16 743 pages x 4 KV heads x 8448 B) read by kernels that do
    nothing else, in forms that are not the decode kernel's own (include/kvx_debug.h) --
    a linear read from one extent; the shuffled page list with 16-byte loads of whole KiB at 2, 4
    and 8 waves per SIMD; the decode kernel's own loads over the shuffled list, the list sorted
    by address, a list drawn from 40 GB of the pool only, pages in address order; and twice the
    pages per wave, whose extra time is what the bytes cost once a launch is under way.  One
    JSON line: microseconds and GB/s per form."""
    import numpy as np
    import torch
    from richengine_amd import kvx

    L = kvx.lib()
    torch.cuda.set_device(0)
    rng = np.random.default_rng(args.seed)
    layout = kvx.Layout(LAYERS, H, D, kvx.INT4, 0.0)
    extent_pages = L.kvx_layout_largest_extent_pages(C.byref(layout))
    page_bytes = L.kvx_layout_bytes_per_model_page(C.byref(layout))
    free, _total = torch.cuda.mem_get_info()
    pool_bytes = args.pool_gb * 1e9 if args.pool_gb > 0 else min(0.8 * free, 256e9)
    extents = max(3, int(pool_bytes // (extent_pages * page_bytes)))
    storage = kvx.Storage(LAYERS, H, D, kvx.INT4, extents * extent_pages, extent_pages, aligned=True)
    storage.allocate_all()
    n_pages = 16743
    small = min(extents, 9)
    lists = {
        "shuffled over the pool": rng.permutation(extents * extent_pages)[:n_pages],
        "the same pages sorted by address": None,
        f"shuffled over {small} extents ({small * extent_pages * page_bytes / 1e9:.0f} GB)":
            rng.permutation(small * extent_pages)[:n_pages],
        "pages in address order": np.arange(n_pages),
        "twice the pages, shuffled over the pool": rng.permutation(extents * extent_pages)[:2 * n_pages],
    }
    lists["the same pages sorted by address"] = np.sort(lists["shuffled over the pool"])
    tables = {name: storage.table(ids.astype(np.uint32)) for name, ids in lists.items()}
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)

    def timed(call):
        for layer in range(2):
            kvx.check(call(layer))
        torch.cuda.synchronize()
        k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        k0.record()
        for it in range(args.kernel_iters):
            call(it % LAYERS)
        k1.record()
        torch.cuda.synchronize()
        return k0.elapsed_time(k1) / args.kernel_iters * 1e3  # microseconds

    def kernel_loads(name, per):
        table = tables[name]
        return timed(lambda layer: L.kvx_calibrate_stream(storage.h, layer, table.data_ptr(), table.numel(),
                                                          per, 1, sink.data_ptr(), stream))

    def form(name, which, per, depth, waves):
        table = tables[name]
        return timed(lambda layer: L.kvx_calibrate_stream_form(storage.h, layer, table.data_ptr(),
                                                               table.numel(), per, which, depth, waves,
                                                               sink.data_ptr(), stream))

    nbytes = n_pages * H * 8448
    rows = []

    def row(what, us, count=n_pages):
        rows.append({"form": what, "us": round(us, 1), "gbs": round(count * H * 8448 / us / 1e3, 0)})

    shuffled = "shuffled over the pool"
    for per in (4, 16):
        row(f"linear read of the same bytes from one extent, {2 * per} pieces of 4 KiB per wave",
            form(shuffled, 2, per, 1, 8))
    for waves in (2, 4, 8):
        row(f"shuffled list, 16-byte loads of whole KiB, one page ahead, {waves} waves per SIMD, 34 pages per wave",
            form(shuffled, 1, 34, 1, waves))
    row("shuffled list, 16-byte loads of whole KiB, two pages ahead, 2 waves per SIMD, 34 pages per wave",
        form(shuffled, 1, 34, 2, 2))
    for per in (16, 34, 64):
        row(f"shuffled list, the decode kernel's loads, 2 waves per SIMD, {per} pages per wave",
            kernel_loads(shuffled, per))
    one = rows[-2]["us"]
    for name in list(lists)[1:4]:
        row(f"{name}, the decode kernel's loads, 34 pages per wave", kernel_loads(name, 34))
    two = kernel_loads("twice the pages, shuffled over the pool", 68)
    row("twice the pages at 68 per wave (the same number of waves), the decode kernel's loads", two,
        2 * n_pages)
    rows.append({"form": "the second half of those bytes: what the list costs once a launch is under way",
                 "us": round(two - one, 1), "gbs": round(nbytes / (two - one) / 1e3, 0)})
    result = {
        "metric": "HBM read rate for one layer of the int4 batch-32 decode step's pages, by request shape",
        "value": rows[0]["gbs"], "unit": "GB/s", "n_gpus": 1, "steps": args.kernel_iters, "warmup": 2,
        "ms_per_step": round(rows[0]["us"] / 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": "calibration: 16 743 pages x 4 KV heads x 8448 B per launch (the headline "
                               "batch's bytes of one layer), pool of %d extents, %.1f GB" %
                               (extents, extents * extent_pages * page_bytes / 1e9),
                   "bytes_per_launch": nbytes, "seed": args.seed},
        "forms": rows,
        "roofline": {"bound": "hbm", "achieved": rows[0]["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(rows[0]["gbs"] / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "stream_linear_kernel (a plain read, no attention)"},
        "cpu_baseline": None,
    }
    storage.close()
    print(json.dumps(result))


def qkv_prepare(args):
    """QKV prepare fused with quantize-on-append (kv_prepare_append), int4 pages, the
    reference's 24 query heads with gates, bf16 norms, 32 rotary pairs: a 2048-token prefill
    chunk per launch (the roofline line: packed rows and rotation tables read, queries and
    pages written), and the one-row step of a batch of 32.  kv_append of ready bf16 chunk
    rows, which the fused kernel replaces together with the prepare kernel in front of it, is
    timed beside both."""
    import numpy as np
    import torch
    from richengine_amd import kvx

    L = kvx.lib()
    torch.cuda.set_device(0)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(args.seed)
    rng = np.random.default_rng(args.seed)
    layout = kvx.Layout(LAYERS, H, D, kvx.INT4, 0.0)
    extent_pages = L.kvx_layout_largest_extent_pages(C.byref(layout))
    storage = kvx.Storage(LAYERS, H, D, kvx.INT4, extent_pages, extent_pages, aligned=True)
    storage.allocate_all()
    ids = rng.permutation(extent_pages).astype(np.uint32)
    pairs, width = 32, (2 * QH + 2 * H) * D
    shape = kvx.QkvShape(QH, pairs, 1, 1, 0.0)
    wq = torch.randn(D, generator=gen, device="cuda").bfloat16()
    wk = torch.randn(D, generator=gen, device="cuda").bfloat16()

    def timed(call):
        call(0)
        torch.cuda.synchronize()
        k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        k0.record()
        for it in range(args.kernel_iters):
            call(it % LAYERS)
        k1.record()
        torch.cuda.synchronize()
        return k0.elapsed_time(k1) / args.kernel_iters

    def case(lanes, committed, tokens):
        rows = tokens
        stride = (tokens + 31) // 32 * 32
        n_pages = (committed + tokens + 31) // 32
        tables = [storage.table(ids[i * n_pages:(i + 1) * n_pages]) for i in range(lanes)]
        packed = torch.randn((lanes, rows, width), generator=gen, device="cuda").bfloat16()
        cos = torch.rand((lanes, rows, pairs), generator=gen, device="cuda")
        sin = torch.rand((lanes, rows, pairs), generator=gen, device="cuda")
        queries = torch.zeros((lanes, H, stride, G, D), dtype=torch.bfloat16, device="cuda")
        chunk_k = torch.randn((lanes, H, stride, D), generator=gen, device="cuda").bfloat16()
        chunk_v = torch.randn((lanes, H, D, stride), generator=gen, device="cuda").bfloat16()
        cp = [kvx.ChunkParams(committed, tokens, stride, n_pages) for _ in range(lanes)]
        fused = timed(lambda layer: kvx.prepare_append(storage, layer, shape, packed, wq, wk, cos, sin,
                                                       queries, stride, tables, cp, rows))
        store = timed(lambda layer: kvx.append(storage, layer, chunk_k, chunk_v, tables, cp,
                                               H * stride * D))
        # what the kernel has to move per row: the query, key and value parts of the packed
        # row (the gate halves belong to the attention epilogue and are not read here), the
        # rotation, the prepared queries and the page bytes
        moved = lanes * tokens * ((QH + 2 * H) * D * 2 + 2 * pairs * 4 + QH * D * 2 + BYTES_PER_TOKEN_LAYER)
        return fused, store, moved

    chunk_ms, chunk_store_ms, chunk_bytes = case(1, 16384, 2048)
    step_ms, step_store_ms, _ = case(BATCH, 4096, 1)
    achieved = chunk_bytes / (chunk_ms * 1e-3) / 1e9
    result = {
        "metric": "qkv prepare + int4 quantize-on-append, 2048-token chunk: tokens/s per layer launch",
        "value": round(2048 / (chunk_ms * 1e-3), 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.kernel_iters, "warmup": 1, "ms_per_step": round(chunk_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 rows, fp32 norm and rotation, int4 pages", "data": "synthetic",
        "config": {"workload": "kv_prepare_append: 24 query heads with gates, 4 KV heads x 256, bf16 "
                               "norms, 32 rotary pairs; one 2048-token chunk after 16384 committed "
                               "tokens per launch",
                   "seed": args.seed},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "prepare_append_wave_kernel<int4, 4, 4> (one wave per head and four rows; bound by its vector instructions)", "bytes_per_launch": chunk_bytes,
                     "ms_per_launch": round(chunk_ms, 4)},
        "kv_append_alone_ms": round(chunk_store_ms, 4),
        "decode_batch32_one_row": {"prepare_append_ms": round(step_ms, 4),
                                   "kv_append_alone_ms": round(step_store_ms, 4)},
        "cpu_baseline": None,
    }
    storage.close()
    if args.cpu_seconds > 0:
        result["cpu_baseline"] = cpu_qkv_prepare(args.seed, args.cpu_seconds)
    print(json.dumps(result))


def shared_prefix(args):
    """Decode attention of 16 sequences that share a 30 016-token prompt prefix (938 pages) and
    hold 64..1024 tokens of their own, int4 pages, one layer per launch: kv_attend_decode_shared
    (the prefix read once for all sequences) beside kv_attend_decode on the same page tables (the
    prefix read once per sequence).  `value` is sequence-steps per second of one layer's
    attention with the shared entry; the KV bytes counted are those of the whole sequences,
    which is what the unshared entry has to read."""
    import numpy as np
    import torch
    from richengine_amd import kvx

    L = kvx.lib()
    torch.cuda.set_device(0)
    rng = np.random.default_rng(args.seed)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(args.seed)
    fmt = {"bf16": kvx.BF16, "int8": kvx.INT8, "int4": kvx.INT4}[args.format]
    bytes_per_token = {"bf16": 4096, "int8": 2080, "int4": BYTES_PER_TOKEN_LAYER}[args.format]
    lanes, shared_pages = 16, 938
    own = [int(t) for t in rng.integers(64, 1025, lanes)]
    own_pages = [(t + 1 + 31) // 32 for t in own]
    layout = kvx.Layout(LAYERS, H, D, fmt, 0.0)
    extent_pages = L.kvx_layout_largest_extent_pages(C.byref(layout))
    storage = kvx.Storage(LAYERS, H, D, fmt, extent_pages, extent_pages, aligned=True)
    storage.allocate_all()
    ids = rng.permutation(extent_pages).astype(np.uint32)
    prefix, first, tables = ids[:shared_pages], shared_pages, []
    for n in own_pages:
        tables.append(storage.table(np.concatenate([prefix, ids[first:first + n]])))
        first += n
    entries = [shared_pages + n for n in own_pages]

    def fill(lane, start, count):
        done = 0
        while done < count:
            n = min(2048, count - done)
            stride = (n + 31) // 32 * 32
            k = torch.randn((H, stride, D), generator=gen, device="cuda").bfloat16()
            v = torch.randn((H, D, stride), generator=gen, device="cuda").bfloat16()
            for layer in range(LAYERS):
                kvx.append(storage, layer, k, v, [tables[lane]],
                           [kvx.ChunkParams(start + done, n, stride, entries[lane])], H * stride * D)
            done += n

    fill(0, 0, shared_pages * 32)
    for lane in range(lanes):
        fill(lane, shared_pages * 32, own[lane] + 1)
    committed = [shared_pages * 32 + t for t in own]
    queries = torch.randn((lanes, H, 1, G, D), generator=gen, device="cuda").bfloat16()
    output = torch.zeros_like(queries)
    prefix_splits = args.verify_splits or kvx.verify_plan([shared_pages * 32], lanes, H, QH, fmt)[0]
    own_splits = kvx.decode_plan(own, H, fmt)
    sp = [kvx.VerifyParams(committed[i], entries[i], kvx.KvLayer(), own_splits[i], own_splits[i], 1, 1, 0.0)
          for i in range(lanes)]
    plain_splits = kvx.decode_plan(committed, H, fmt)
    pp = [kvx.VerifyParams(committed[i], entries[i], kvx.KvLayer(), plain_splits[i], plain_splits[i], 1, 1,
                           0.0) for i in range(lanes)]
    ws = torch.empty(max(kvx.attend_shared_workspace_bytes(storage, sp, prefix_splits, QH),
                         kvx.attend_workspace_bytes(storage, pp, QH)) + 4096, dtype=torch.uint8, device="cuda")

    def timed(call):
        call(0)
        torch.cuda.synchronize()
        k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        k0.record()
        for it in range(args.kernel_iters):
            call(it % LAYERS)
        k1.record()
        torch.cuda.synchronize()
        return k0.elapsed_time(k1) / args.kernel_iters

    shared_ms = timed(lambda layer: kvx.attend_decode_shared(storage, layer, QH, queries, output, tables, sp,
                                                             shared_pages, prefix_splits, 1, ws))
    plain_ms = timed(lambda layer: kvx.attend_decode(storage, layer, QH, queries, output, tables, pp, 1, ws))
    logical = sum(c + 1 for c in committed) * bytes_per_token
    physical = (shared_pages * 32 + sum(t + 1 for t in own)) * bytes_per_token
    result = {
        "metric": args.format + " decode attention over a shared prefix, 16 sequences x 30 016 shared tokens: "
                  "sequence-steps/s of one layer",
        "value": round(lanes / (shared_ms * 1e-3), 1), "unit": "sequence-steps/s", "n_gpus": 1,
        "steps": args.kernel_iters, "warmup": 1, "ms_per_step": round(shared_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.format + " pages, bf16 / fp16 MFMA, fp32 accumulate", "data": "synthetic",
        "config": {"workload": "kv_attend_decode_shared: 16 sequences, 938 shared pages, 64..1024 own "
                               "tokens each, 4 KV heads x 256, 24 query heads, one layer per call",
                   "format": args.format, "prefix_splits": int(prefix_splits), "seed": args.seed},
        # Decode is bandwidth-bound: the bytes the entry has to read are the shared pages once
        # and every sequence's own pages (`physical`), over the time of the whole call.
        "roofline": {"bound": "hbm", "achieved": round(physical / (shared_ms * 1e-3) / 1e9, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(physical / (shared_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "bytes_per_launch": physical,
                     "mfma_tflops": round(4 * D * QH * sum(c + 1 for c in committed) /
                                          (shared_ms * 1e-3) / 1e12, 1),
                     "traffic": None, "kernel": "split kernels over the shared pages (stacked rows) and over the "
                                                "sequences' own pages + shared_merge_kernel",
                     "ms_per_launch": round(shared_ms, 4)},
        "unshared_ms": round(plain_ms, 4),
        "kv_bytes_logical": logical, "kv_bytes_physical": physical,
        "logical_kv_gbs_shared": round(logical / (shared_ms * 1e-3) / 1e9, 1),
        "logical_kv_gbs_unshared": round(logical / (plain_ms * 1e-3) / 1e9, 1),
        "cpu_baseline": None,
    }
    storage.close()
    if args.cpu_seconds > 0 and args.format == "int4":
        # one sequence of the 16 (the oracle has no shared form: every sequence walks its whole table)
        spent = cpu_lane(int(committed[0]), args.seed)
        result["cpu_baseline"] = {
            "value": 1.0 / spent, "unit": "sequence-steps/s", "cores": 1, "kind": "port", **host_cpus(),
            "sample": f"one sequence of the 16 ({int(committed[0]) + 1} tokens), one layer: append 1 token + "
                      f"decode attention over its whole table, {spent:.1f} s of scalar C++ oracle"}
    print(json.dumps(result))


def control_plane(args):
    """The host side of a serving step at batch 32, no GPU work: the prefix page cache and the
    sequence records (kvx_prefix_*, kvx_sequence_*) over an accounting-only storage of the
    benchmark's layout.  32 requests of 16 384 prompt tokens whose first 8192 are shared are
    admitted (match, restore, then chunks of 2048 tokens: pages, publish, page list), decode
    `--steps` x 32 steps of one token (pages, publish, page list per sequence), run as many
    16-row tree-verify steps (pages for the tree, publish what was accepted, truncate) and
    end (every block evicted).  The calls go through ctypes with arguments built beforehand;
    the cost of an empty ctypes call is measured beside them and `value` is the decode step
    with that taken off.  The CPU baseline is the oracle's restatement of the reference's
    cache (Python over the oracle's page pool) on a shorter run of the same steps."""
    import random
    import time
    from richengine_amd import kvx

    L = kvx.lib()
    rng = random.Random(args.seed)
    sequences, shared, prompt_tokens, chunk = 32, 8192, 16384, 2048
    steps = max(32 * args.steps, 32)
    most = prompt_tokens + 2 * steps * 6 + 64
    pages = sequences * ((most + 31) // 32 + 1)
    extent_pages = 1024
    pages = (pages + extent_pages - 1) // extent_pages * extent_pages
    prefix_tokens = [rng.randrange(150000) for _ in range(shared)]
    streams = [prefix_tokens + [rng.randrange(150000) for _ in range(most - shared)]
               for _ in range(sequences)]

    def product():
        storage = kvx.Storage(LAYERS, H, D, kvx.INT4, pages, extent_pages, accounting=True)
        pool = kvx.Pool(storage, extent_pages)
        prefix = kvx.Prefix(pool)
        records = kvx.Sequences(pool, prefix)
        tokens = [(C.c_uint32 * most)(*t) for t in streams]
        blocks, matched = (C.c_uint64 * (prompt_tokens // 32))(), C.c_uint32()
        view, released = kvx.SequencePages(), C.c_uint32()
        S, P = records.h, prefix.h
        calls = 0

        def ok(rc):
            if rc:
                raise kvx.KvxError(rc, kvx.lib().kvx_last_error().decode())

        now = time.perf_counter_ns
        # the cost of a ctypes call that does nothing
        t0 = now()
        for _ in range(200000):
            L.kvx_prefix_generation(P)
        empty_ns = (now() - t0) / 200000
        admit_ns, admit_calls, hit_blocks = [], [], []
        for i in range(sequences):
            t0, n = now(), 3
            ok(L.kvx_sequence_begin(S, i + 1))
            L.kvx_prefix_match(P, tokens[i], prompt_tokens, blocks, len(blocks), C.byref(matched))
            if matched.value:
                ok(L.kvx_sequence_restore(S, i + 1, blocks[matched.value - 1]))
                n += 1
            committed = 32 * matched.value
            while committed < prompt_tokens:
                committed = min(prompt_tokens, committed + chunk)
                ok(L.kvx_sequence_ensure_tokens(S, i + 1, committed))
                ok(L.kvx_sequence_publish(S, i + 1, tokens[i], prompt_tokens, committed))
                ok(L.kvx_sequence_view(S, i + 1, C.byref(view)))
                n += 3
            admit_ns.append(now() - t0)
            admit_calls.append(n)
            hit_blocks.append(matched.value)
        length = [prompt_tokens] * sequences
        t0 = now()
        for _ in range(steps):
            for i in range(sequences):
                length[i] += 1
                ok(L.kvx_sequence_ensure_tokens(S, i + 1, length[i]))
                ok(L.kvx_sequence_publish(S, i + 1, tokens[i], length[i], length[i]))
                ok(L.kvx_sequence_view(S, i + 1, C.byref(view)))
        decode_ns = (now() - t0) / steps
        accepted = [[rng.randrange(1, 6) for _ in range(sequences)] for _ in range(steps)]
        t0 = now()
        for step in range(steps):
            for i in range(sequences):
                ok(L.kvx_sequence_ensure_tokens(S, i + 1, length[i] + 16))
                length[i] += accepted[step][i]
                ok(L.kvx_sequence_publish(S, i + 1, tokens[i], length[i], length[i]))
                ok(L.kvx_sequence_truncate(S, i + 1, length[i], C.byref(released)))
                ok(L.kvx_sequence_view(S, i + 1, C.byref(view)))
        verify_ns = (now() - t0) / steps
        resident = L.kvx_prefix_block_count(P)
        t0 = now()
        for i in range(sequences):
            ok(L.kvx_sequence_end(S, i + 1))
        block, evicted = C.c_uint64(), 0
        while L.kvx_prefix_eviction_candidate(P, 0, C.byref(block)) == 1:
            ok(L.kvx_prefix_erase(P, block.value))
            evicted += 1
        end_ns = now() - t0
        snapshot = pool.snapshot()
        assert evicted == resident and snapshot.pages_active == 0 and snapshot.pages_prefix == 0
        records.close(); prefix.close(); pool.close(); storage.close()
        return {"empty_ns": empty_ns, "admit_ns": admit_ns, "admit_calls": admit_calls,
                "hit_blocks": hit_blocks, "decode_ns": decode_ns, "verify_ns": verify_ns,
                "end_ns": end_ns, "evicted": evicted, "final_length": length}

    def port(budget_s):
        from oracle import kvoracle as ko
        from oracle import prefix_oracle as po
        import numpy as np
        KL = ko.lib()

        class Pages:   # the oracle's page pool behind the three calls the cache makes
            def __init__(self):
                self.h = KL.ko_pool_create(pages, 100, extent_pages, extent_pages, 0xFFFFFFFF)
                self.pages, self.extent_pages = pages, extent_pages
            def acquire(self, count):
                out = np.zeros(max(count, 1), dtype=np.uint32)
                if KL.ko_pool_acquire(self.h, count, ko.ptr(out)) != count:
                    raise po.OracleError("nomem")
                return [int(x) for x in out[:count]]
            def retain(self, page, prefix_owner):
                if KL.ko_pool_retain(self.h, page, int(prefix_owner)):
                    raise po.OracleError("state")
            def release(self, page, prefix_owner):
                if KL.ko_pool_release(self.h, page, int(prefix_owner)):
                    raise po.OracleError("state")

        pool = Pages()
        prefix = po.PrefixCache(pool, pages)
        records = po.SequenceCache(pool, prefix, pool.acquire)
        started = time.perf_counter()
        admitted = 0
        t0 = time.perf_counter_ns()
        for i in range(sequences):
            records.begin(i + 1)
            found = []
            prefix.extend_match(found, streams[i][:prompt_tokens])
            if found:
                records.restore(i + 1, found[-1])
            committed = 32 * len(found)
            while committed < prompt_tokens:
                committed = min(prompt_tokens, committed + chunk)
                records.ensure_tokens(i + 1, committed)
                records.publish(i + 1, streams[i][:prompt_tokens], committed)
            admitted += 1
        admit_ns = (time.perf_counter_ns() - t0) / admitted
        length = [prompt_tokens] * sequences
        done = 0
        t0 = time.perf_counter_ns()
        while done < steps and time.perf_counter() - started < budget_s:
            for i in range(sequences):
                length[i] += 1
                records.ensure_tokens(i + 1, length[i])
                records.publish(i + 1, streams[i][:length[i]], length[i])
            done += 1
        decode_ns = (time.perf_counter_ns() - t0) / max(done, 1)
        return {"admit_us": admit_ns / 1e3, "decode_step_us": decode_ns / 1e3, "steps": done}

    for _ in range(max(args.warmup, 0) and 1):
        product()
    m = product()
    per_step_calls = 3 * sequences
    net_decode_us = (m["decode_ns"] - per_step_calls * m["empty_ns"]) / 1e3
    warm = [i for i in range(sequences) if m["hit_blocks"][i]]
    cold_us = m["admit_ns"][0] / 1e3
    warm_us = sum(m["admit_ns"][i] for i in warm) / max(len(warm), 1) / 1e3
    baseline = port(args.cpu_seconds) if args.cpu_seconds > 0 else None
    result = {
        "metric": "kv_control_plane_decode_step_us", "value": round(net_decode_us, 2), "unit": "us per step of 32 sequences",
        "n_gpus": 1, "steps": steps, "warmup": 1 if args.warmup else 0,
        "ms_per_step": round(m["decode_ns"] / 1e6, 5), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "host", "data": "synthetic",
        "config": {"workload": "host control plane at batch 32: prefix page cache and sequence records over "
                               "accounting-only storage, 32 x 16384-token prompts sharing 8192 tokens, then "
                               "one-token decode steps and 16-row tree-verify steps",
                   "layers": LAYERS, "kv_heads": H, "head_dim": D, "format": "int4", "pool_pages": pages},
        "roofline": None,
        "calls": {
            "empty_ctypes_call_ns": round(m["empty_ns"], 1),
            "decode_step_us_with_call_overhead": round(m["decode_ns"] / 1e3, 2),
            "decode_step_calls": per_step_calls,
            "tree_verify_step_us_with_call_overhead": round(m["verify_ns"] / 1e3, 2),
            "tree_verify_step_calls": 4 * sequences,
            "admission_cold_us": round(cold_us, 1), "admission_cold_calls": m["admit_calls"][0],
            "admission_shared_prefix_us": round(warm_us, 1),
            "admission_shared_prefix_calls": m["admit_calls"][-1],
            "admission_matched_blocks": m["hit_blocks"][-1],
            "end_and_evict_us": round(m["end_ns"] / 1e3, 1), "blocks_evicted": m["evicted"],
        },
        "cpu_baseline": None if baseline is None else {
            "value": round(baseline["decode_step_us"], 1), "unit": "us per step of 32 sequences", "cores": 1,
            "kind": "port",
            "sample": f"oracle/prefix_oracle.py over the oracle's page pool: the same admissions "
                      f"({baseline['admit_us']:.0f} us each on average) and {baseline['steps']} of the decode steps"},
    }
    print(json.dumps(result))


def chunked_prefill(args):
    """Chunked prefill with prefix reuse: batch 4, a 2048-token chunk per sequence appended onto a
    shared 16384-token prefix (the prefix pages are the same physical pages in every
    sequence's table), bf16 or fp8 pages.  A step = per layer and sequence, quantize +
    scatter of the chunk, then causal attention of its 2048 rows over prefix + chunk.
    The attention kernel's line carries the MFMA roofline (useful flops = 4 x D x
    query heads x sum over rows of the tokens the row sees)."""
    import numpy as np
    import torch
    from richengine_amd import kvx

    L = kvx.lib()
    torch.cuda.set_device(0)
    rng = np.random.default_rng(args.seed)
    fmt = {"bf16": kvx.BF16, "fp8": kvx.FP8, "int8": kvx.INT8, "int4": kvx.INT4}[args.format]
    peak = 2500.0  # bf16 and fp16 MFMA (the one-byte formats multiply as fp16)
    sequences, prefix, chunk = 4, 16384, args.prefill_chunk
    prefix_pages, chunk_pages = prefix // 32, chunk // 32
    total = prefix_pages + sequences * chunk_pages
    layout = kvx.Layout(LAYERS, H, D, fmt, 0.0)
    extent_pages = L.kvx_layout_largest_extent_pages(C.byref(layout))
    extents = -(-total // extent_pages)
    storage = kvx.Storage(LAYERS, H, D, fmt, extents * extent_pages, extent_pages, aligned=True)
    storage.allocate_all()
    ids = rng.permutation(extents * extent_pages)[:total].astype(np.uint32)
    shared = ids[:prefix_pages]
    tables = [storage.table(np.concatenate([shared, ids[prefix_pages + s * chunk_pages:
                                                        prefix_pages + (s + 1) * chunk_pages]]))
              for s in range(sequences)]
    entries = prefix_pages + chunk_pages
    gen = torch.Generator(device="cuda")
    gen.manual_seed(args.seed)

    def rows(shape):  # N(0,1); fp8 pages take values clipped to the e4m3 range of the scaled codes
        return torch.randn(shape, generator=gen, device="cuda").clamp_(-6, 6).bfloat16()

    for done in range(0, prefix, 2048):
        k, v = rows((H, 2048, D)), rows((H, D, 2048))
        for layer in range(LAYERS):
            kvx.append(storage, layer, k, v, [tables[0]], [kvx.ChunkParams(done, 2048, 2048, entries)],
                       H * 2048 * D)
    chunk_k = [rows((H, chunk, D)) for _ in range(sequences)]
    chunk_v = [rows((H, D, chunk)) for _ in range(sequences)]
    queries = [rows((H, chunk, G, D)) for _ in range(sequences)]
    # One stream, output and workspace per sequence: the sequences of a batch are
    # independent, and the 1536 waves of one sequence's launch leave half of the
    # SIMDs idle in their second round on the formats that run one wave per SIMD.
    # Launches of other sequences on other streams fill that round.
    # --prefill-streams 0: the whole batch per layer in one kv_append and one
    # kv_attend_prefill_batch call on one stream (every sequence's tiles in the same launch).
    if args.prefill_streams is None:
        args.prefill_streams = 0 if args.format == "int4" else 4
    batched = args.prefill_streams == 0
    n_streams = max(1, min(args.prefill_streams, sequences))
    streams = [torch.cuda.Stream() for _ in range(n_streams)] if n_streams > 1 else [None]
    outputs = [torch.zeros_like(queries[0]) for _ in range(n_streams)]
    output = outputs[0]
    # the split count fills the GPU's wave slots with the launch it is for: one sequence's tiles, or
    # (batched) every sequence's
    splits = kvx.prefill_plan(prefix, chunk, H, QH, fmt)
    batch_splits = kvx.prefill_plan(prefix, chunk, H, QH, fmt, sequences=sequences)
    cp = kvx.ChunkParams(prefix, chunk, chunk, entries)
    pp = kvx.PrefillParams(prefix, chunk, chunk, entries, kvx.KvLayer(), splits, 0.0)
    batch_pp = kvx.PrefillParams(prefix, chunk, chunk, entries, kvx.KvLayer(), batch_splits, 0.0)
    workspaces = [torch.empty(kvx.prefill_workspace_bytes(storage, chunk, QH, splits) + 4096, dtype=torch.uint8,
                              device="cuda") for _ in range(n_streams)]
    workspace = workspaces[0]
    if batched:
        all_k, all_v, all_q = torch.stack(chunk_k), torch.stack(chunk_v), torch.stack(queries)
        all_out = torch.zeros_like(all_q)
        all_ws = torch.empty(sequences * kvx.prefill_workspace_bytes(storage, chunk, QH, batch_splits) + 4096,
                             dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()

    def step():
        if batched:
            for layer in range(LAYERS):
                kvx.append(storage, layer, all_k, all_v, tables, [cp] * sequences, H * chunk * D)
                kvx.attend_prefill_batch(storage, layer, QH, all_q, all_out, tables, [batch_pp] * sequences,
                                         H * chunk * G * D, all_ws)
            return
        # a sequence's layers follow one another on its stream, as they do in a model
        for layer in range(LAYERS):
            for s in range(sequences):
                lane = s % n_streams
                handle = streams[lane].cuda_stream if streams[lane] is not None else None
                kvx.append(storage, layer, chunk_k[s], chunk_v[s], [tables[s]], [cp], H * chunk * D,
                           stream=handle)
                kvx.attend_prefill(storage, layer, QH, queries[s], outputs[lane], tables[s], pp,
                                   workspaces[lane], stream=handle)

    steps, warmup = min(args.steps, 5), min(args.warmup, 1)
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    iters = max(2, args.kernel_iters // 4)
    k0.record()
    for it in range(iters):
        kvx.attend_prefill(storage, it % LAYERS, QH, queries[it % sequences], output,
                           tables[it % sequences], pp, workspace)
    k1.record()
    torch.cuda.synchronize()
    single_ms = k0.elapsed_time(k1) / iters
    flops = 4 * D * QH * sum(prefix + r + 1 for r in range(chunk))
    kernel_ms, launch_sequences = single_ms, 1
    if batched:
        # the launch the step runs: every sequence's tiles in one kv_attend_prefill_batch call
        k0.record()
        for it in range(iters):
            kvx.attend_prefill_batch(storage, it % LAYERS, QH, all_q, all_out, tables, [batch_pp] * sequences,
                                     H * chunk * G * D, all_ws)
        k1.record()
        torch.cuda.synchronize()
        kernel_ms, launch_sequences = k0.elapsed_time(k1) / iters, sequences
    flops *= launch_sequences
    achieved = flops / (kernel_ms * 1e-3) / 1e12
    result = {
        "metric": f"{args.format} chunked prefill ({chunk}-token chunks onto a shared 16384-token prefix, "
                  "batch 4): prefill tokens/s",
        "value": round(sequences * chunk * steps / wall, 1), "unit": "tokens/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": round(wall * 1e3 / steps, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"bf16": "bf16 pages, bf16 MFMA", "fp8": "fp8e4m3 pages, fp16 MFMA",
                  "int8": "int8 pages, fp16 MFMA", "int4": "int4 pages, bf16 MFMA"}[args.format] +
                 ", fp32 accumulate",
        "data": "synthetic",
        "config": {"workload": "BASELINE configs[3]: chunked prefill with a shared prefix, batch 4, "
                               f"{chunk}-row chunks over 16384 + {chunk} tokens, 16 layers: quantize + scatter "
                               "of the chunk, then causal attention per layer and sequence",
                   "batch": sequences, "layers": LAYERS, "format": args.format,
                   "splits": int(batch_splits if batched else splits), "splits_of_one_launch": int(splits),
                   "streams": 0 if batched else n_streams,
                   "calls": "kv_attend_prefill_batch, one per layer" if batched
                            else "kv_attend_prefill, one per layer and sequence",
                   "seed": args.seed},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 1), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(achieved / peak, 4), "traffic": None,
                     "kernel": ("kv_attend_prefill_batch of one layer: every sequence's tiles in one launch of "
                                "the split kernel (prefill_int4_kernel or group_wide_kernel)" if batched else
                                "kv_attend_prefill of one sequence and layer: the split kernel (prefill_int4_kernel "
                                "or group_wide_kernel) and, with several splits, the merge behind it"),
                     "flops_per_launch": flops, "ms_per_launch": round(kernel_ms, 4),
                     "sequences_per_launch": launch_sequences,
                     "one_sequence_ms_per_launch": round(single_ms, 4)},
        "cpu_baseline": None,
    }
    storage.close()
    if args.cpu_seconds > 0:
        result["cpu_baseline"] = cpu_prefill(args.seed, args.format, prefix, chunk, args.cpu_seconds)
    print(json.dumps(result))


def single_decode(args):
    """One sequence, context 32768, int4, 16 layers, contiguous page table: a step appends one
    token and runs decode attention in every layer (kv_append_attend_decode, one call per
    layer).  The 16 calls are captured once in a HIP graph and a step is one replay: a lone
    sequence leaves the GPU nothing to overlap the launches with, so the gaps between them
    are what a graph removes.  Every replay stores the same token and attends the same
    32769 tokens.  Eager steps (the same calls issued one by one) are timed beside it."""
    import numpy as np
    import torch
    from richengine_amd import kvx

    L = kvx.lib()
    torch.cuda.set_device(0)
    context = args.uniform_context or 32768
    n_pages = (context + 1 + 31) // 32
    layout = kvx.Layout(LAYERS, H, D, kvx.INT4, 0.0)
    extent_pages = L.kvx_layout_largest_extent_pages(C.byref(layout))
    extents = -(-n_pages // extent_pages)
    storage = kvx.Storage(LAYERS, H, D, kvx.INT4, extents * extent_pages, extent_pages, aligned=True)
    storage.allocate_all()
    table = storage.table(np.arange(n_pages, dtype=np.uint32))
    gen = torch.Generator(device="cuda")
    gen.manual_seed(args.seed)
    for done in range(0, context, 2048):
        n = min(2048, context - done)
        stride = (n + 31) // 32 * 32
        k = torch.randn((H, stride, D), generator=gen, device="cuda").bfloat16()
        v = torch.randn((H, D, stride), generator=gen, device="cuda").bfloat16()
        for layer in range(LAYERS):
            kvx.append(storage, layer, k, v, [table], [kvx.ChunkParams(done, n, stride, n_pages)],
                       H * stride * D)
    chunk_k = torch.randn((1, H, 32, D), generator=gen, device="cuda").bfloat16()
    chunk_v = torch.randn((1, H, D, 32), generator=gen, device="cuda").bfloat16()
    queries = torch.randn((1, H, 1, G, D), generator=gen, device="cuda").bfloat16()
    output = torch.zeros_like(queries)
    splits = kvx.decode_plan([context], H)[0]
    if args.pages_per_split:
        splits = min(max(1, -(-n_pages // args.pages_per_split)), 512)
    vp = [kvx.VerifyParams(context, n_pages, kvx.KvLayer(), splits, splits, 1, 1, 0.0)]
    vp_arr = (kvx.VerifyParams * 1)(*vp)
    ws_bytes = kvx.attend_workspace_bytes(storage, vp, QH) + (1 << 20)
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    table_arr = (C.c_void_p * 1)(table.data_ptr())

    def layers(stream):
        for layer in range(LAYERS):
            rc = L.kv_append_attend_decode(storage.h, layer, chunk_k.data_ptr(), chunk_v.data_ptr(),
                                           H * 32 * D, 32, QH, queries.data_ptr(), output.data_ptr(),
                                           table_arr, vp_arr, 1, 1, workspace.data_ptr(), ws_bytes, stream)
            if rc:
                kvx.check(rc)

    def timed(run, count):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(count):
            run()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / count

    eager_stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    for _ in range(max(args.warmup, 1)):
        layers(eager_stream)
    eager_s = timed(lambda: layers(eager_stream), args.steps)
    eager_out = output.clone()

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layers(C.c_void_p(side.cuda_stream))  # every kernel loaded before the capture
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            layers(C.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(max(args.warmup, 1)):
        graph.replay()
    # Replays between eager work and synchronisations, each checked against the eager result.
    for _ in range(3):
        output.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(output, eager_out), "a graph replay differs from the eager step"
        layers(eager_stream)
    step_s = timed(graph.replay, args.steps)

    def time_kernel(call):
        call(0)
        torch.cuda.synchronize()
        k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        k0.record()
        for it in range(args.kernel_iters):
            call(it % LAYERS)
        k1.record()
        torch.cuda.synchronize()
        return k0.elapsed_time(k1) / args.kernel_iters

    split_ms = time_kernel(lambda layer: L.kv_attend_split(
        storage.h, layer, QH, queries.data_ptr(), table_arr, vp_arr, 1, None, 1, workspace.data_ptr(),
        ws_bytes, eager_stream))
    merge_ms = time_kernel(lambda layer: L.kv_attend_merge(
        storage.h, QH, output.data_ptr(), vp_arr, 1, 1, workspace.data_ptr(), ws_bytes, eager_stream))
    layer_bytes = (context + 1) * BYTES_PER_TOKEN_LAYER
    value = layer_bytes * LAYERS / step_s / 1e9
    achieved = layer_bytes / (split_ms * 1e-3) / 1e9
    result = {
        "metric": "int4 paged decode attn, one sequence of 32768 tokens: KV GB/s per step",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "int4 pages, bf16 MFMA, fp32 accumulate", "data": "synthetic",
        "config": {"workload": "BASELINE configs[1]: single-sequence int4 decode, batch 1, context "
                               f"{context}, 16 layers, contiguous page table: 1-token append + split-K "
                               "paged attention per layer; a step = one replay of the HIP graph of the "
                               "16 per-layer calls",
                   "batch": 1, "layers": LAYERS, "context": context, "splits": int(splits),
                   "pages_per_split": -(-n_pages // int(splits)), "seed": args.seed},
        "pct_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "decode_tokens_per_s": round(1 / step_s, 1),
        "us_per_layer": round(step_s * 1e6 / LAYERS, 2),
        "eager_ms_per_step": round(eager_s * 1e3, 4),
        "eager_us_per_layer": round(eager_s * 1e6 / LAYERS, 2),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "decode_int4_kernel (split kernel of paged decode attention), one layer per launch",
                     "bytes_per_launch": layer_bytes, "ms_per_launch": round(split_ms, 4),
                     "merge_ms_per_launch": round(merge_ms, 4)},
        "cpu_baseline": None,
    }
    storage.close()
    if args.cpu_seconds > 0:
        spent = cpu_lane(context, args.seed)
        result["cpu_baseline"] = {
            "value": layer_bytes / spent / 1e9, "unit": "GB/s", "cores": 1, "kind": "port", **host_cpus(),
            "sample": f"the sequence itself, one layer of the 16: append 1 token + decode attention over "
                      f"{context + 1} tokens, {spent:.1f} s of scalar C++ oracle"}
    print(json.dumps(result))


def decode_layout(args):
    """One-row decode attention over the reference's other shipped layouts (2 KV heads x 8 x 128
    and 8 x 4 x 64, runtime/ops/PagedAttention.cpp:66-115): 32 sequences of 8192 tokens, one
    layer per call, split counts from kvx_decode_plan_for.  `value` is KV bytes per second of
    kv_attend_decode (split + reduce); the roofline leg times the split kernel alone."""
    import numpy as np
    import torch
    from richengine_amd import kvx

    torch.cuda.set_device(0)
    heads, group, dim = {"hd128": (2, 8, 128), "hd64": (8, 4, 64)}[args.layout]
    fmt = {"bf16": kvx.BF16, "fp8": kvx.FP8, "int8": kvx.INT8, "int4": kvx.INT4}[args.format]
    per_token = heads * {"bf16": 4 * dim, "fp8": 2 * dim + 8, "int8": 2 * dim + 8, "int4": dim + 8}[args.format]
    lanes, context = 32, 8192
    n_pages = (context + 31) // 32
    query_heads = heads * group
    pool_pages = 8192 * (-(-lanes * n_pages // 8192))
    storage = kvx.Storage(1, heads, dim, fmt, pool_pages, 8192, aligned=True)
    storage.allocate_all()
    rng = np.random.default_rng(args.seed)
    ids = rng.permutation(lanes * n_pages).astype(np.uint32)
    tables = [storage.table(ids[i * n_pages:(i + 1) * n_pages]) for i in range(lanes)]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(args.seed)
    for i in range(lanes):
        for done in range(0, context, 2048):
            k = torch.randn((heads, 2048, dim), generator=gen, device="cuda").bfloat16()
            v = torch.randn((heads, dim, 2048), generator=gen, device="cuda").bfloat16()
            kvx.append(storage, 0, k, v, [tables[i]], [kvx.ChunkParams(done, 2048, 2048, n_pages)],
                       heads * 2048 * dim)
    q = torch.randn((lanes, heads, 1, group, dim), generator=gen, device="cuda").bfloat16()
    out = torch.zeros_like(q)
    splits = kvx.decode_plan_for(storage, [context - 1] * lanes)
    dp = [kvx.VerifyParams(context - 1, n_pages, kvx.KvLayer(), splits[i], splits[i], 1, 1, 0.0)
          for i in range(lanes)]
    ws = torch.empty(kvx.attend_workspace_bytes(storage, dp, query_heads), dtype=torch.uint8, device="cuda")

    def timed(fn, n):
        for _ in range(max(args.warmup, 1)):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n * 1e-3

    call_s = timed(lambda: kvx.attend_decode(storage, 0, query_heads, q, out, tables, dp, 1, ws), args.steps)
    split_s = timed(lambda: kvx.attend_split(storage, 0, query_heads, q, tables, dp, None, 1, ws), args.kernel_iters)
    merge_s = timed(lambda: kvx.attend_merge(storage, query_heads, out, dp, 1, ws), args.kernel_iters)
    kv_bytes = lanes * context * per_token
    value = kv_bytes / call_s / 1e9
    achieved = kv_bytes / split_s / 1e9
    result = {
        "metric": "decode_kv_read_GBps", "value": round(value, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": max(args.warmup, 1), "ms_per_step": round(call_s * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"int4": "int4 codes -> bf16 MFMA", "int8": "int8 codes -> bf16 MFMA",
                  "fp8": "e4m3 -> fp16 MFMA", "bf16": "bf16 MFMA"}[args.format],
        "data": "synthetic",
        "config": {"workload": f"one-row decode attention, {heads} KV heads x {group} x {dim} ({args.layout}), "
                               f"{args.format} pages, batch {lanes} x {context} tokens, one layer per call",
                   "splits_per_sequence": int(splits[0]), "seed": args.seed},
        "pct_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                     "kernel": "attend_split_small_wave_kernel (a wave per sequence, KV head and split)",
                     "bytes_per_launch": kv_bytes, "ms_per_launch": round(split_s * 1e3, 4),
                     "reduce_ms_per_launch": round(merge_s * 1e3, 4)},
        "cpu_baseline": None,
    }
    storage.close()
    if args.cpu_seconds > 0:
        from oracle import kvoracle as ko
        oracle_fmt = {"bf16": ko.BF16, "fp8": ko.FP8, "int8": ko.INT8, "int4": ko.INT4}[args.format]
        spent = cpu_lane(context - 1, args.seed, H=heads, G=group, D=dim, fmt=oracle_fmt)
        result["cpu_baseline"] = {
            "value": context * per_token / spent / 1e9, "unit": "GB/s", "cores": 1, "kind": "port", **host_cpus(),
            "sample": f"one of the 32 sequences: append 1 token + decode attention over {context} tokens, "
                      f"{spent:.2f} s of scalar C++ oracle"}
    print(json.dumps(result))


def prefill_layout(args):
    """A chunk of chunked prefill over the reference's other shipped layouts (2 KV heads x 8 x 128,
    8 x 4 x 64) and two with smaller groups of query heads (2 x 4 x 128, 4 x 2 x 128): `--prefill-chunk`
    rows (2048 by default) over 16 384 tokens of history, one sequence, one layer per call, splits
    from kvx_prefill_plan_for.  Timed on a history that ends on a page boundary, where the tiles that
    begin in the same page share a workgroup and a staged page, and on the same history plus one
    token, where every tile runs on its own.  `value` is the matrix-core rate of the first."""
    import numpy as np
    import torch
    from richengine_amd import kvx

    torch.cuda.set_device(0)
    heads, group, dim = {"hd128": (2, 8, 128), "hd64": (8, 4, 64), "k2q4d128": (2, 4, 128),
                         "k4q2d128": (4, 2, 128)}[args.layout]
    fmt = {"bf16": kvx.BF16, "fp8": kvx.FP8, "int8": kvx.INT8, "int4": kvx.INT4}[args.format]
    rows, history = args.prefill_chunk, 16384
    query_heads = heads * group
    n_pages = (history + 1 + rows + 31) // 32
    storage = kvx.Storage(1, heads, dim, fmt, 8192, 8192, aligned=True)
    storage.allocate_all()
    table = storage.table(np.random.default_rng(args.seed).permutation(n_pages).astype(np.uint32))
    gen = torch.Generator(device="cuda")
    gen.manual_seed(args.seed)
    for done in range(0, n_pages * 32, 2048):
        n = min(2048, n_pages * 32 - done)
        k = torch.randn((heads, n, dim), generator=gen, device="cuda").bfloat16()
        v = torch.randn((heads, dim, n), generator=gen, device="cuda").bfloat16()
        kvx.append(storage, 0, k, v, [table], [kvx.ChunkParams(done, n, n, n_pages)], heads * n * dim)
    q = torch.randn((heads, rows, group, dim), generator=gen, device="cuda").bfloat16()
    out = torch.zeros_like(q)
    layout = kvx.Layout(1, heads, dim, fmt, 0.0)

    def timed(committed):
        splits = kvx.prefill_plan_for(storage, committed, rows, query_heads)
        together = kvx.lib().kvx_debug_prefill_tiles_together(C.byref(layout), query_heads, committed, rows, splits)
        params = kvx.PrefillParams(committed, rows, rows, n_pages, kvx.KvLayer(), splits, 0.0)
        ws = torch.empty(kvx.prefill_workspace_bytes(storage, rows, query_heads, splits), dtype=torch.uint8,
                         device="cuda")
        call = lambda: kvx.attend_prefill(storage, 0, query_heads, q, out, table, params, ws)
        for _ in range(max(args.warmup, 1)):
            call()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            call()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps * 1e-3, int(splits), int(together)

    aligned_s, aligned_splits, together = timed(history)
    alone_s, alone_splits, alone_together = timed(history + 1)
    flops = 4.0 * dim * query_heads * rows * (history + (rows + 1) / 2)
    peak = 2500.0   # the tiles multiply bf16 (fp16 on fp8 pages): 2.5 PFLOP/s dense either way
    achieved = flops / aligned_s / 1e12
    result = {
        "metric": "prefill_attention_TFLOPs", "value": round(achieved, 1), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": max(args.warmup, 1), "ms_per_step": round(aligned_s * 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp16 MFMA" if args.format == "fp8" else "bf16 MFMA", "data": "synthetic",
        "config": {"workload": f"chunked prefill attention, {heads} KV heads x {group} x {dim} ({args.layout}), "
                               f"{args.format} pages, {rows} rows over {history} tokens, one sequence, one layer "
                               f"per call", "splits": aligned_splits, "tiles_per_workgroup": together,
                   "seed": args.seed},
        "one_token_past_the_page_boundary": {"ms_per_step": round(alone_s * 1e3, 4), "splits": alone_splits,
                                             "tiles_per_workgroup": alone_together,
                                             "TFLOPs": round(flops / alone_s / 1e12, 1)},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 1), "peak": peak, "unit": "TFLOP/s",
                     "frac": round(achieved / peak, 4), "traffic": None,
                     "kernel": "prefill_group_small_kernel / prefill_split_small_kernel + prefill_reduce_kernel "
                               "(the call; the split kernel is all but a few microseconds of it)",
                     "flops_per_launch": flops, "ms_per_launch": round(aligned_s * 1e3, 4)},
        "cpu_baseline": None,
    }
    storage.close()
    print(json.dumps(result))


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: the KV path of this build has no multi-GPU leg "
              "(run with --gpus 1)", file=sys.stderr)
        sys.exit(2)
    if args.workload != "decode":
        from richengine_amd import kvx
        if not os.path.exists(kvx.LIB_PATH):
            from richengine_amd import build as kvx_build
            kvx_build.build(verbose=False)
        if args.workload == "qkv-prepare":
            return qkv_prepare(args)
        if args.workload == "stream-ceiling":
            return stream_ceiling(args)
        if args.workload == "decode-single":
            return single_decode(args)
        if args.workload == "shared-prefix":
            return shared_prefix(args)
        if args.workload == "control-plane":
            return control_plane(args)
        if args.workload == "decode-layout":
            if args.layout not in ("hd128", "hd64"):
                sys.exit("decode-layout takes --layout hd128 or hd64")
            return decode_layout(args)
        if args.workload == "prefill-layout":
            return prefill_layout(args)
        return tree_verify(args) if args.workload == "tree-verify" else chunked_prefill(args)
    import numpy as np
    import torch
    from richengine_amd import kvx

    if not os.path.exists(kvx.LIB_PATH):
        from richengine_amd import build as kvx_build
        kvx_build.build(verbose=False)
    L = kvx.lib()
    torch.cuda.set_device(0)
    rng = np.random.default_rng(args.seed)

    # ---- pool -----------------------------------------------------------------
    layout = kvx.Layout(LAYERS, H, D, kvx.INT4, 0.0)
    extent_pages = L.kvx_layout_largest_extent_pages(C.byref(layout))
    page_bytes = L.kvx_layout_bytes_per_model_page(C.byref(layout))
    extent_bytes = extent_pages * page_bytes
    free, _total = torch.cuda.mem_get_info()
    pool_bytes = args.pool_gb * 1e9 if args.pool_gb > 0 else min(0.8 * free, 256e9)
    extents = max(1, int(pool_bytes // extent_bytes))
    contexts = rng.integers(512, 32769, BATCH)
    if args.uniform_context:
        contexts[:] = args.uniform_context
    total_steps = args.warmup + args.steps + args.kernel_iters + 8
    lane_pages = [(int(c) + total_steps + 31) // 32 for c in contexts]
    while extents * extent_pages < sum(lane_pages):
        extents += 1
    storage = kvx.Storage(LAYERS, H, D, kvx.INT4, extents * extent_pages, extent_pages, aligned=True)
    storage.allocate_all()
    pool_pages = extents * extent_pages
    ids_all = (np.arange(pool_pages) if args.contiguous else rng.permutation(pool_pages))
    ids = ids_all[:sum(lane_pages)].astype(np.uint32)
    tables, first = [], 0
    for n in lane_pages:
        tables.append(storage.table(ids[first:first + n]))
        first += n

    # ---- history: quantize-on-append through the library ----------------------
    gen = torch.Generator(device="cuda")
    gen.manual_seed(args.seed)
    for lane, ctx in enumerate(contexts):
        ctx, done = int(ctx), 0
        while done < ctx:
            n = min(2048, ctx - done)
            stride = (n + 31) // 32 * 32
            k = torch.randn((H, stride, D), generator=gen, device="cuda", dtype=torch.float32).bfloat16()
            v = torch.randn((H, D, stride), generator=gen, device="cuda", dtype=torch.float32).bfloat16()
            for layer in range(LAYERS):
                kvx.append(storage, layer, k, v, [tables[lane]],
                           [kvx.ChunkParams(done, n, stride, lane_pages[lane])], H * stride * D)
            done += n
    torch.cuda.synchronize()

    # ---- step buffers -----------------------------------------------------------
    chunk_k = torch.randn((BATCH, H, 32, D), generator=gen, device="cuda").bfloat16()
    chunk_v = torch.randn((BATCH, H, D, 32), generator=gen, device="cuda").bfloat16()
    queries = torch.randn((BATCH, H, 1, G, D), generator=gen, device="cuda").bfloat16()
    output = torch.zeros_like(queries)
    committed = [int(c) for c in contexts]

    def lane_params():
        ap = [kvx.ChunkParams(committed[i], 1, 32, lane_pages[i]) for i in range(BATCH)]
        vp = []
        plan = kvx.decode_plan(committed, H)
        for i in range(BATCH):
            s = plan[i]
            if args.pages_per_split:
                pages = (committed[i] + 1 + 31) // 32
                s = min(max(1, -(-pages // args.pages_per_split)), 128)
            vp.append(kvx.VerifyParams(committed[i], lane_pages[i], kvx.KvLayer(), s, s, 1, 1, 0.0))
        return ap, vp

    _, vp_max = lane_params()
    ws_bytes = 2 * kvx.attend_workspace_bytes(storage, vp_max, QH) + (1 << 20)
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda")
    table_arr = (C.c_void_p * BATCH)(*[t.data_ptr() for t in tables])
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    lane_stride = H * 32 * D
    hidden = packed = None
    if args.hidden != "none":
        hidden = torch.zeros((BATCH, 1, QH, D), dtype=torch.bfloat16, device="cuda")
        if args.hidden == "gate":
            packed = torch.randn((BATCH, 1, (2 * QH + 2 * H) * D), generator=gen, device="cuda").bfloat16()

    qkv_shape = qkv_packed = None
    if args.prepare:
        args.separate_append = True
        qkv_shape = kvx.QkvShape(QH, 32, 1, 1, 0.0)
        qkv_packed = packed if packed is not None else torch.randn(
            (BATCH, 1, (2 * QH + 2 * H) * D), generator=gen, device="cuda").bfloat16()
        norm_q = torch.randn(D, generator=gen, device="cuda").bfloat16()
        norm_k = torch.randn(D, generator=gen, device="cuda").bfloat16()
        rope_cos = torch.rand((BATCH, 1, 32), generator=gen, device="cuda")
        rope_sin = torch.rand((BATCH, 1, 32), generator=gen, device="cuda")

    def attend(layer, vp_arr):
        if hidden is None:
            return L.kv_attend_decode(storage.h, layer, QH, queries.data_ptr(), output.data_ptr(),
                                      table_arr, vp_arr, BATCH, 1, workspace.data_ptr(), ws_bytes, stream)
        return L.kv_attend_verify_hidden(storage.h, layer, QH, queries.data_ptr(), output.data_ptr(),
                                         table_arr, vp_arr, BATCH, None, 1, workspace.data_ptr(),
                                         ws_bytes, packed.data_ptr() if packed is not None else None,
                                         hidden.data_ptr(), stream)

    def step():
        ap, vp = lane_params()
        ap_arr = (kvx.ChunkParams * BATCH)(*ap)
        vp_arr = (kvx.VerifyParams * BATCH)(*vp)
        for layer in range(LAYERS):
            if not args.separate_append:
                # one call per layer: the token is stored by the attention kernel itself
                if hidden is None:
                    rc = L.kv_append_attend_decode(storage.h, layer, chunk_k.data_ptr(), chunk_v.data_ptr(),
                                                   lane_stride, 32, QH, queries.data_ptr(),
                                                   output.data_ptr(), table_arr, vp_arr, BATCH, 1,
                                                   workspace.data_ptr(), ws_bytes, stream)
                else:
                    rc = L.kv_append_attend_decode_hidden(
                        storage.h, layer, chunk_k.data_ptr(), chunk_v.data_ptr(), lane_stride, 32, QH,
                        queries.data_ptr(), output.data_ptr(), table_arr, vp_arr, BATCH, 1,
                        workspace.data_ptr(), ws_bytes, packed.data_ptr() if packed is not None else None,
                        hidden.data_ptr(), stream)
                if rc:
                    kvx.check(rc)
                continue
            if args.prepare:
                rc = L.kv_prepare_append(storage.h, layer, C.byref(qkv_shape), qkv_packed.data_ptr(),
                                         norm_q.data_ptr(), norm_k.data_ptr(), rope_cos.data_ptr(),
                                         rope_sin.data_ptr(), queries.data_ptr(), 1, table_arr, ap_arr,
                                         BATCH, 1, 15, stream)
            else:
                rc = L.kv_append(storage.h, layer, chunk_k.data_ptr(), chunk_v.data_ptr(), table_arr,
                                 ap_arr, BATCH, lane_stride, 15, stream)
            if rc:
                kvx.check(rc)
            rc = attend(layer, vp_arr)
            if rc:
                kvx.check(rc)
        for i in range(BATCH):
            committed[i] += 1

    if args.copy_calibration_pages:
        # Spare pages at the end of the shuffled order: read N pages, write N pages.
        n = min(args.copy_calibration_pages, (pool_pages - sum(lane_pages)) // 2)
        order = ids_all[sum(lane_pages):sum(lane_pages) + 2 * n]
        storage.copy_pages([(int(order[i]), int(order[n + i])) for i in range(n)])
        torch.cuda.synchronize()
        print(f"copy calibration: {n} pages, {n * page_bytes} bytes read and as many written",
              file=sys.stderr)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    kv_bytes = 0
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        kv_bytes += sum(c + 1 for c in committed) * BYTES_PER_TOKEN_LAYER * LAYERS
        step()
    stop.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    gpu_ms = start.elapsed_time(stop)
    ms_per_step = wall * 1e3 / args.steps
    value = kv_bytes / wall / 1e9

    # ---- dominant kernel: the split kernel of decode attention, one layer of the
    # batch per launch.  Same inputs as a step's attention; events sit on the
    # launch stream.  The merge kernel and both together are timed the same way.
    _, vp = lane_params()
    vp_arr = (kvx.VerifyParams * BATCH)(*vp)
    launch_bytes = sum(c + 1 for c in committed) * BYTES_PER_TOKEN_LAYER

    def time_attend(which):
        # "both": the attend call as a step issues it; "split" / "merge": the two dispatches
        # as calls of their own (kv_attend_split, kv_attend_merge) over the same lanes
        def call(layer):
            if which == "both":
                return attend(layer, vp_arr)
            if which == "split":
                return L.kv_attend_split(storage.h, layer, QH, queries.data_ptr(), table_arr, vp_arr,
                                         BATCH, None, 1, workspace.data_ptr(), ws_bytes, stream)
            return L.kv_attend_merge(storage.h, QH, output.data_ptr(), vp_arr, BATCH, 1,
                                     workspace.data_ptr(), ws_bytes, stream)
        for layer in range(2):
            kvx.check(call(layer))
        torch.cuda.synchronize()
        k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        k0.record()
        for it in range(args.kernel_iters):
            call(it % LAYERS)
        k1.record()
        torch.cuda.synchronize()
        return k0.elapsed_time(k1) / args.kernel_iters

    both_ms = time_attend("both")
    kernel_ms = time_attend("split")
    merge_ms = time_attend("merge")
    achieved = launch_bytes / (kernel_ms * 1e-3) / 1e9
    traffic = profiled_traffic()

    # ---- what the access pattern streams at: the same pages through the split kernel's
    # own loads with no arithmetic behind them (kvx_calibrate_stream), 32 pages per wave
    # as the plan gives the long lanes.
    live = [(c + 1 + 31) // 32 for c in committed]
    all_entries = torch.cat([tables[i][:live[i]] for i in range(BATCH)]).contiguous()
    sink = torch.zeros(1, dtype=torch.int32, device="cuda")

    def time_stream(per, heads):
        def call(layer):
            return L.kvx_calibrate_stream(storage.h, layer, all_entries.data_ptr(), all_entries.numel(),
                                          per, heads, sink.data_ptr(), stream)
        for layer in range(2):
            kvx.check(call(layer))
        torch.cuda.synchronize()
        k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        k0.record()
        for it in range(args.kernel_iters):
            call(it % LAYERS)
        k1.record()
        torch.cuda.synchronize()
        return k0.elapsed_time(k1) / args.kernel_iters

    stream_bytes = all_entries.numel() * 32 * BYTES_PER_TOKEN_LAYER
    stream_ms = {per: time_stream(per, 1) for per in (16, 32, 64)}
    stream4_ms = {per: time_stream(per, 4) for per in (16, 32, 64)}

    result = {
        "metric": "int4 paged decode attn: KV GB/s (% HBM peak) + decode tokens/s, bs=32",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int4 pages, bf16 MFMA, fp32 accumulate",
        "data": "synthetic",
        "config": {
            "workload": "BASELINE configs[2]: batched mixed-length int4 decode, batch 32, contexts "
                        "U[512,32768], 16 layers, 4 KV heads x 256, 24 query heads, 1-token append "
                        "+ split-K paged attention per layer",
            "batch": BATCH, "layers": LAYERS, "context_tokens_total": int(sum(committed)),
            "pool_gb": round(extents * extent_bytes / 1e9, 1), "extents": extents,
            "page_order": "contiguous" if args.contiguous else "seed-shuffled",
            "seed": args.seed,
            **({"entries": ("kv_append_attend_decode_hidden" if not args.separate_append else
                            ("kv_prepare_append" if args.prepare else "kv_append") + " + " +
                            ("kv_attend_verify_hidden" if args.hidden != "none" else "kv_attend_decode")),
                "hidden": args.hidden}
               if args.hidden != "none" or args.prepare else {}),
        },
        "pct_hbm_peak": round(100 * value / HBM_PEAK_GBS, 2),
        "decode_tokens_per_s": round(BATCH * args.steps / wall, 1),
        "gpu_ms_per_step": round(gpu_ms / args.steps, 4),
        "roofline": {
            "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
            "kernel": "decode_int4_quad_kernel (split kernel of paged decode attention, workgroups of four waves), one layer of the batch per launch",
            "bytes_per_launch": launch_bytes, "ms_per_launch": round(kernel_ms, 4),
            "merge_ms_per_launch": round(merge_ms, 4), "split_plus_merge_ms": round(both_ms, 4),
            "split_plus_merge_gbs": round(launch_bytes / (both_ms * 1e-3) / 1e9, 1),
            "stream_ceiling": {
                "what": "the split kernel's page loads alone (kvx_calibrate_stream) over the same pages, "
                        "whole pages counted",
                "bytes_per_launch": stream_bytes,
                "gbs_by_pages_per_wave": {str(per): round(stream_bytes / (ms * 1e-3) / 1e9, 1)
                                          for per, ms in stream_ms.items()},
                "ms_by_pages_per_wave": {str(per): round(ms, 4) for per, ms in stream_ms.items()},
                "gbs_four_heads_per_workgroup": {str(per): round(stream_bytes / (ms * 1e-3) / 1e9, 1)
                                                 for per, ms in stream4_ms.items()},
            },
        },
    }
    storage.close()
    if args.cpu_seconds > 0:
        result["cpu_baseline"] = cpu_baseline(contexts, args.seed, args.cpu_seconds)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
