#!/usr/bin/env python3
"""Benchmark of the int8-KV decode layer call on one MI355X.

One step = one layer call of the hot path over one synthetic dynamic batch:
quantise/append of the step's new K/V rows, decode attention over the int8 cache
(token-range kernel + combine) and, for the mixed workload, the chunked-prefill
tile.  Inputs are resident in HBM before the timed region.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3]

Prints one JSON line.  `value` = algorithmic decode bytes of the batch divided by
the whole step time (GB/s).  The K timed steps are K layer calls recorded once into a HIP
graph; the graph is replayed R >= 10 times back to back with an event between the replays,
and the step time is the MEDIAN replay divided by K (`replays_us_per_layer` also gives the
first and the fastest; `--eager` times host-launched kernels instead, which is also
reported as `us_per_layer_eager` (sustained) and `us_per_layer_eager_from_idle`).  `roofline` prices the dominant kernel alone (the
token-range decode kernel, named by the library) in the same regime: a graph of K launches
of that kernel, replayed and timed the same way on the stream it is launched on; the
figure of an event-separated launch loop is given beside it (`stages_us`).
`cpu_baseline` is the CPU oracle (quantise/append + decode attention) on a bounded sample of the same batch.

The cache has `--layers` layers (default 8) and timed call i works on layer i mod layers, as the layers of a model
follow each other: two calls on the same layer are then separated by the cache bytes of all the other layers (gigabytes),
so nothing of a layer's cache is left in the 256 MB memory-side cache when its turn comes again.  `same_layer` gives
the figure of the regime in which every call re-reads one layer, for comparison.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published


def read_traffic(workload, kernel):
    """HBM bytes per launch of the decode kernel from the rocprofv3 --pmc summary under profiles/ (counters
    cannot be read from inside this process), or None when the summary is absent or is of another kernel."""
    path = os.path.join(ROOT, "profiles", "decode_attention_%s_traffic.txt" % workload)
    try:
        text = open(path).read()
    except OSError:
        return None
    if kernel not in text:
        return None
    for line in text.splitlines():
        if line.startswith("traffic_bytes_per_launch:"):
            return float(line.split(":", 1)[1])
    return None


def cpu_baseline(oracle, bt, lay, q, k, v, cache_host, scale_host, budget_s=2.0):
    """The oracle's step -- quantise/append of the new K/V rows, then decode attention -- over the first sequences of
    the batch (decode sequences, one new row each), sized to the time budget.  `cache_host` / `scale_host`: a cache of
    one layer in the layout `lay`."""
    kw = dict(cache_stride_s=lay.stride_s, cache_stride_l=lay.stride_l, cache_stride_h=lay.stride_h,
              cache_stride_kv=lay.stride_kv, cachestarts_stride_b=bt.cachestarts_stride_b)
    d = bt.head_dim
    per_tok = bt.num_kv_heads * (2 * d + 2 * (d // 8) * 2)

    def run(nseq):
        kvstarts = bt.kvstarts[:nseq + 1]
        rows = int(bt.seqstarts[nseq])
        t0 = time.perf_counter()
        oracle.kv_cache_quantize(k[:rows], v[:rows], bt.seqstarts[:nseq + 1], bt.cachestarts, bt.start_pos[:nseq], 0,
                                 bt.num_kv_heads, d, bt.page_size, cache=cache_host, scale=scale_host, **kw)
        t1 = time.perf_counter()
        oracle.decode_attention(q, cache_host, scale_host, bt.cachestarts, kvstarts, nseq, bt.num_heads,
                                bt.num_kv_heads, d, bt.attn_scale, 0, bt.page_size, **kw)
        t2 = time.perf_counter()
        tokens = int(bt.kv_lens[:nseq].sum())
        return t2 - t0, t1 - t0, tokens * per_tok + 2 * nseq * bt.num_heads * d * 2, tokens

    n0 = max(1, min(bt.decoding_batches, 4))
    dt, _, nbytes, tokens = run(n0)  # also warms the pages
    rate = tokens / max(dt, 1e-6)
    cum = np.cumsum(bt.kv_lens[:bt.decoding_batches])
    # as many sequences as one pass of about a second covers, then passes until the budget is spent
    nseq = int(min(bt.decoding_batches, max(n0, np.searchsorted(cum, rate * 1.0) + 1)))
    times, appends = [], []
    t_all = time.perf_counter()
    while not times or (time.perf_counter() - t_all < budget_s and len(times) < 50):
        dt, dt_append, nbytes, tokens = run(nseq)
        times.append(dt)
        appends.append(dt_append)
    dt = float(np.median(times))
    cores = oracle.num_threads()
    return {"value": nbytes / dt / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": "quantise/append of the new rows + decode attention of the first %d of %d sequences (%d kv tokens): "
                      "median of %d passes of %.2f s, of which the append %.1f ms (%.0f core-seconds in all)" % (
                          nseq, bt.decoding_batches, tokens, len(times), dt, float(np.median(appends)) * 1e3,
                          sum(times) * cores),
            "us_per_layer_extrapolated": dt * 1e6 * bt.decode_kv_tokens / max(tokens, 1)}


def extras(torch, ops, dev, bt, replay_times):
    """Microseconds per call, in the replayed-graph regime of the rest of the line, of the kernels either side of
    the layer call: RoPE on the step's query and key rows, RoPE fused with the quantise/append, the append alone,
    and kv_cache_reorder / kv_cache_invert_reorder of 64 pages of a (4 layers, 8 kv heads, 128 channels) cache."""
    lk = dev.layout_kwargs()
    kw = dict(theta=10000.0, rotary_dim=bt.head_dim, batch=bt.batch, max_seqlen=bt.max_seqlen)
    rq, rk = torch.empty_like(dev.query), torch.empty_like(dev.new_key)
    n_new = int(bt.q_lens.sum())
    res = {"new_tokens": n_new}
    res["rope_us"] = float(np.median(replay_times(lambda st: ops.rotary_position_embedding(
        dev.query, dev.new_key, dev.start_pos, dev.seqstarts, rq, rk, stream=st, **kw))))
    res["append_us"] = float(np.median(replay_times(lambda st: ops.key_value_cache(
        dev.new_key, dev.new_value, dev.seqstarts, dev.cachestarts, dev.start_pos, dev.cache, dev.scale, batch=bt.batch,
        max_seqlen=bt.max_seqlen, num_layer=bt.num_layer, layer_idx=bt.layer_idx, num_kv_heads=bt.num_kv_heads,
        head_dim=bt.head_dim, stream=st, **lk))))
    res["rope_append_fused_us"] = float(np.median(replay_times(lambda st: ops.rope_key_value_cache(
        dev.query, dev.new_key, dev.new_value, dev.start_pos, dev.seqstarts, dev.cachestarts, rq, None, dev.cache,
        dev.scale, num_layer=bt.num_layer, layer_idx=bt.layer_idx, stream=st, **lk, **kw))))
    # the fused call rewrote this step's cache rows from rotated keys: put the plain ones back
    ops.key_value_cache(dev.new_key, dev.new_value, dev.seqstarts, dev.cachestarts, dev.start_pos, dev.cache, dev.scale,
                        batch=bt.batch, max_seqlen=bt.max_seqlen, num_layer=bt.num_layer, layer_idx=bt.layer_idx,
                        num_kv_heads=bt.num_kv_heads, head_dim=bt.head_dim, **lk)
    layers, heads, d, group, pool_pages = 4, 8, 128, 8, 256
    t_page, sb = 128, d // group * 2
    tok = pool_pages * t_page
    src = [0, 2 * heads * tok * d, heads * tok * d, tok * d, d, 1, 0, 2 * heads * tok * sb, heads * tok * sb, tok * sb, sb, 1]
    pcb, psb = t_page * heads * 2 * layers * d, t_page * heads * 2 * layers * sb
    dst = [0, d, layers * d, 2 * layers * d, heads * 2 * layers * d, 1, 0, sb, layers * sb, 2 * layers * sb, heads * 2 * layers * sb, 1]
    src[0], src[6] = pcb, psb
    cache = torch.randint(0, 255, (layers, 2, heads, tok, d), dtype=torch.uint8, device="cuda")
    scale = torch.randint(0, 255, (layers, 2, heads, tok, sb), dtype=torch.uint8, device="cuda")
    ids = torch.randperm(pool_pages, device="cuda")[:64].to(torch.int64)
    outer = torch.empty(64 * (pcb + psb), dtype=torch.uint8, device="cuda")
    pk = dict(layers=layers, kv_heads=heads, tokens=t_page, head_dim=d, group_size=group, tp_rank=0, tp_size=1)
    moved = 64 * (pcb + psb)
    res["reorder_bytes_moved"] = moved
    res["kv_cache_reorder_us"] = float(np.median(replay_times(lambda st: ops.kv_cache_reorder(
        cache, scale, ids, src, dst, outer_mem=outer, stream=st, **pk))))
    inv_src = [pcb] + dst[1:6] + [psb] + dst[7:]
    res["kv_cache_invert_reorder_us"] = float(np.median(replay_times(lambda st: ops.kv_cache_invert_reorder(
        outer, ids, inv_src, src, kv_cache=cache, kv_scale=scale, stream=st, **pk))))
    return res


def rope_sweep_bench(torch, pkg, steps, replays):
    """--rope-sweep: RoPE followed by the quantise/append as two kernels against the fused kernel, by the number of
    new tokens of a step (32 query / 8 kv heads of 128; 128 sequences of one token, then 16 sequences of equal length).
    A graph of `steps` calls replayed `replays` times back to back, median replay."""
    wl, harness, ops = pkg.workloads, pkg.harness, pkg.ops
    hq, hkv, d = 32, 8, 128
    side = torch.cuda.Stream()

    def timed(call):
        call(torch.cuda.current_stream())
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for _ in range(steps):
                    call(side)
            graph.replay()
            side.synchronize()
            evs = [torch.cuda.Event(enable_timing=True) for _ in range(replays + 1)]
            evs[0].record(side)
            for r in range(replays):
                graph.replay()
                evs[r + 1].record(side)
            side.synchronize()
        return float(np.median([evs[r].elapsed_time(evs[r + 1]) * 1e3 / steps for r in range(replays)]))

    rows = []
    for n_tok, nseq in ((128, 128), (512, 16), (1024, 16), (2048, 16), (4096, 16), (8192, 16), (16384, 16)):
        bt, rng = wl.custom_batch(3, hq, hkv, d, 1, [], prefill_q_lens=[n_tok // nseq] * nseq, prefill_prior=[64] * nseq)
        dev = harness.DeviceBatch(bt)
        q, k, v = wl.step_inputs(bt, rng)
        dev.set_step_inputs(q, k, v)
        lk = dev.layout_kwargs()
        kw = dict(theta=10000.0, rotary_dim=d, batch=bt.batch, max_seqlen=bt.max_seqlen)
        rq, rk = torch.empty_like(dev.query), torch.empty_like(dev.new_key)

        def rope(st):
            ops.rotary_position_embedding(dev.query, dev.new_key, dev.start_pos, dev.seqstarts, rq, rk, stream=st, **kw)

        def append(st):
            ops.key_value_cache(rk, dev.new_value, dev.seqstarts, dev.cachestarts, dev.start_pos, dev.cache, dev.scale,
                                batch=bt.batch, max_seqlen=bt.max_seqlen, num_layer=1, layer_idx=0, num_kv_heads=hkv,
                                head_dim=d, stream=st, **lk)

        def fused(st):
            ops.rope_key_value_cache(dev.query, dev.new_key, dev.new_value, dev.start_pos, dev.seqstarts, dev.cachestarts,
                                     rq, rk, dev.cache, dev.scale, num_layer=1, layer_idx=0, stream=st, **lk, **kw)

        rows.append({"new_tokens": n_tok, "sequences": nseq, "rope_us": timed(rope), "append_us": timed(append),
                     "two_kernels_us": timed(lambda st: (rope(st), append(st))), "fused_us": timed(fused)})
    print(json.dumps({
        "metric": "RoPE + quantise/append of a step's new rows, microseconds per call", "unit": "us",
        "higher_is_better": False, "n_gpus": 1, "steps": steps, "data": "synthetic",
        "dtype": "fp16 rows, int8 cache", "config": {"workload": "rope-sweep: 32 q / 8 kv heads of 128"},
        "value": rows[0]["fused_us"], "sweep": rows}))


def chunk_bench(torch, pkg, spec, steps, replays):
    """--chunks: the prefill stage on a batch of short chunks (a few query tokens per sequence over a long history, no
    decode sequences), once on the tile kernel (no workspace) and once with the workspace that routes it to the decode
    step's MFMA kernel.  A graph of `steps` stage calls replayed `replays` times back to back, median replay."""
    wl, harness, ops = pkg.workloads, pkg.harness, pkg.ops
    c = dict(hq=32, hkv=8, d=128, seqs=64, qmin=2, qmax=8, prior=2048, mode=1)
    c.update({k: int(v) for k, v in (kv.split("=") for kv in spec.split(","))})
    q_lens = np.random.default_rng(5).integers(c["qmin"], c["qmax"] + 1, c["seqs"]).tolist()
    bt, rng = wl.custom_batch(11, num_heads=c["hq"], num_kv_heads=c["hkv"], head_dim=c["d"], cache_mode=c["mode"],
                              dec_kv_lens=[], prefill_q_lens=q_lens, prefill_prior=[c["prior"]] * c["seqs"], outliers=True)
    dev = harness.DeviceBatch(bt)
    dev.fill_history(rng, max_rows=1 << 15)
    q, k, v = wl.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    kw = dict(attn_scale=bt.attn_scale, is_causal=True, batch=bt.batch, decoding_batches=0, max_seqlen=bt.max_seqlen,
              max_kvlen=bt.max_kvlen, layer_idx=bt.layer_idx, num_heads=c["hq"], num_kv_heads=c["hkv"], head_dim=c["d"],
              **dev.layout_kwargs())
    ws_bytes = ops.prefill_workspace_size(bt.batch, 0, bt.max_seqlen, bt.max_kvlen, c["hq"], c["hkv"], c["d"])
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev.device)
    stream, side = torch.cuda.current_stream(), torch.cuda.Stream()

    def timed(workspace):
        def call(st):
            ops.prefill_attention(dev.query, dev.output, dev.cache, dev.scale, dev.seqstarts, dev.kvstarts, dev.cachestarts,
                                  workspace=workspace, stream=st, **kw)
        call(stream)
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for _ in range(steps):
                    call(side)
            graph.replay()
            side.synchronize()
            evs = [torch.cuda.Event(enable_timing=True) for _ in range(replays + 1)]
            evs[0].record(side)
            for r in range(replays):
                graph.replay()
                evs[r + 1].record(side)
            side.synchronize()
        return float(np.median([evs[r].elapsed_time(evs[r + 1]) * 1e3 / steps for r in range(replays)]))

    tile_us = timed(None)
    tile_out = dev.output.clone()
    chunk_us = timed(ws) if ws_bytes else None
    diff = float((dev.output.float() - tile_out.float()).abs().max()) if ws_bytes else None
    cache_bytes = int(sum(int(x) for x in bt.kv_lens)) * c["hkv"] * (2 * c["d"] + c["d"] // 2)
    print(json.dumps({
        "metric": "prefill stage on short chunks, microseconds per call", "unit": "us", "higher_is_better": False,
        "n_gpus": 1, "steps": steps, "data": "synthetic", "dtype": "int8 KV cache, fp16 in/out, fp32 accumulate",
        "config": {"workload": "chunks(%s)" % spec, "sequences": c["seqs"], "query_tokens": [c["qmin"], c["qmax"]],
                   "prior_tokens": c["prior"], "columns_per_kv_head": int(bt.max_seqlen) * (c["hq"] // c["hkv"]),
                   "cache_bytes": cache_bytes},
        "tile_kernel_us": tile_us, "decode_kernel_path_us": chunk_us, "value": chunk_us if chunk_us else tile_us,
        "decode_kernel_path_gbs": cache_bytes / (chunk_us * 1e-6) / 1e9 if chunk_us else None,
        "workspace_bytes": ws_bytes, "max_abs_difference_between_the_two": diff}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="C3", choices=["C2", "C3", "C3m0", "C4", "C5"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--eager", action="store_true", help="time host-launched kernels only (no HIP graph)")
    ap.add_argument("--ranges", type=int, default=0, help="token ranges for decode (0 = planned)")
    ap.add_argument("--replays", type=int, default=12, help="timed replays of the K-step graph (at least 10)")
    ap.add_argument("--layers", type=int, default=8,
                    help="layers of the cache; timed call i works on layer i mod layers (1 = every call re-reads one layer)")
    ap.add_argument("--two-streams", action="store_true",
                    help="mixed steps through forward(stream, side_stream, fork, join): the decode stage on a second "
                         "stream beside the prefill stage")
    ap.add_argument("--no-same-layer", action="store_true",
                    help="skip the comparison run in which every call re-reads layer 0 (profile runs: every launch of the "
                         "trace is then one of the rotating regime)")
    ap.add_argument("--layout", default="l2shd", choices=["l2shd", "sl2hd", "lhs2d"],
                    help="order of the cache tensor: (L,2,S,H,D), (S,L,2,H,D) or (L,H,S,2,D)")
    ap.add_argument("--custom", default="",
                    help="a decode-only batch instead of --workload, e.g. 'hq=8,hkv=1,d=128,batch=64,kvmin=1024,"
                         "kvmax=4096,mode=1,layout=lhs2d' (kv lengths uniform in [kvmin, kvmax], seed 7, outlier channels)")
    ap.add_argument("--chunks", default="",
                    help="instead of a layer call: the prefill stage on a batch of short chunks, e.g. 'hq=32,hkv=8,d=128,"
                         "seqs=64,qmin=2,qmax=8,prior=2048', on the tile kernel and on the decode step's kernel")
    ap.add_argument("--extras", action="store_true",
                    help="also time the kernels either side of the layer call on this batch's new tokens (RoPE alone, "
                         "RoPE fused with the append) and a 64-page kv_cache_reorder; reported under `extras`")
    ap.add_argument("--rope-sweep", action="store_true",
                    help="instead of a layer call: RoPE + append as two kernels against the fused kernel, by new tokens")
    ap.add_argument("--calibration-copy-mib", type=int, default=0,
                    help="also run one plain device copy of this many MiB (known traffic, for scaling rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (the path shards by kv head "
              "with no exchange between GPUs)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    pkg = entry.load_package()
    if not os.path.exists(pkg._lib.LIB_PATH):
        entry.build()
    wl, harness, ops = pkg.workloads, pkg.harness, pkg.ops
    torch.cuda.set_device(0)

    if args.chunks:
        chunk_bench(torch, pkg, args.chunks, args.steps, max(10, args.replays))
        return
    if args.rope_sweep:
        rope_sweep_bench(torch, pkg, args.steps, max(10, args.replays))
        return
    if args.custom:
        c = dict(hq=32, hkv=8, d=128, batch=64, kvmin=1024, kvmax=4096, mode=1, layout=args.layout)
        c.update({k: (v if k == "layout" else int(v)) for k, v in (kv.split("=") for kv in args.custom.split(","))})
        lens = np.random.default_rng(7).integers(c["kvmin"], c["kvmax"] + 1, c["batch"])
        bt, rng = wl.custom_batch(7, c["hq"], c["hkv"], c["d"], c["mode"], lens.tolist(), outliers=True,
                                  num_layer=max(1, args.layers), layout=c["layout"])
        bt.name = "custom(%s)" % args.custom
    else:
        bt, rng = wl.make_batch(args.workload, layout=args.layout, num_layer=max(1, args.layers))
    n_layers = bt.num_layer
    dev = harness.DeviceBatch(bt)
    # context already in the cache: quantised from seeded fp16 rows by the HIP append kernel into layer 0; the other
    # layers hold copies of it at their own addresses
    dev.fill_history(rng, max_rows=1 << 15)
    for layer in range(1, n_layers):
        dev.copy_layer(0, layer)
    q, k, v = wl.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    layer_ops = [dev.make_operator(specify_decoding_multi_block=1, layer_idx=layer) for layer in range(n_layers)]
    op = layer_ops[0]
    for other in layer_ops[1:]:
        other.set_workspace(op.workspace)
    calls = {"n": 0}

    def next_layer():
        """Layer of the next call: 0, 1, ..., layers - 1, 0, ... in the order the calls are issued or recorded."""
        layer = calls["n"] % n_layers
        calls["n"] += 1
        return layer
    if args.ranges:
        plan = ops.decode_plan(bt.decoding_batches, bt.num_heads, bt.num_kv_heads, bt.head_dim, bt.max_kvlen,
                               ranges_hint=args.ranges)
    else:
        plan = ops.decode_plan(bt.decoding_batches, bt.num_heads, bt.num_kv_heads, bt.head_dim, bt.max_kvlen)
    stream = torch.cuda.current_stream()

    def step():
        rc = layer_ops[next_layer()].forward(stream)
        if rc != 0:
            raise RuntimeError("forward() returned %d" % rc)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # Host-launched kernels: K timed calls bracketed by synchronisations (the chip starts them from idle: its first
    # launches after a synchronisation run slower, about a millisecond in all), and K more calls timed by two events
    # behind K calls that were enqueued without a synchronisation in between (the sustained rate of a loop that
    # keeps the queue filled).
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    eager_from_idle_s = (time.perf_counter() - t0) / args.steps
    ev_a, ev_b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(args.steps):
        step()
    ev_a.record(stream)
    for _ in range(args.steps):
        step()
    ev_b.record(stream)
    torch.cuda.synchronize()
    eager_s = ev_a.elapsed_time(ev_b) * 1e-3 / args.steps
    step_s, launch = eager_from_idle_s, "one launch per kernel from the host (eager), timed from idle"
    replays = max(10, args.replays)
    ws = op.workspace
    if ws is None or ws.numel() < int(plan.workspace_size):  # --ranges asked for more ranges than the operator plans
        ws = torch.empty(int(plan.workspace_size), dtype=torch.uint8, device=dev.device)
    side = torch.cuda.Stream()

    def replay_times(record):
        """`record(stream)` enqueues the K launches to time; they are captured once into a HIP graph, the graph is
        replayed twice untimed and then `replays` times back to back with an event between the replays.  Returns the
        per-launch microseconds of every timed replay, in order."""
        side.wait_stream(stream)
        with torch.cuda.stream(side):
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for _ in range(args.steps):
                    record(side)
            graph.replay()
            graph.replay()
            side.synchronize()
            evs = [torch.cuda.Event(enable_timing=True) for _ in range(replays + 1)]
            evs[0].record(side)
            for r in range(replays):
                graph.replay()
                evs[r + 1].record(side)
            side.synchronize()
        stream.wait_stream(side)
        return [evs[r].elapsed_time(evs[r + 1]) * 1e3 / args.steps for r in range(replays)]

    def summary(ts):
        return {"median": float(np.median(ts)), "min": float(np.min(ts)), "first": float(ts[0]), "max": float(np.max(ts))}

    side2 = torch.cuda.Stream() if args.two_streams else None
    fork_ev, join_ev = torch.cuda.Event(), torch.cuda.Event()
    if args.two_streams:
        fork_ev.record(stream)
        join_ev.record(stream)
        torch.cuda.synchronize()

    def forward_on(st):
        if args.two_streams:
            rc = layer_ops[next_layer()].forward_streams(st, side2, fork_ev, join_ev)
        else:
            rc = layer_ops[next_layer()].forward(st)
        if rc != 0:
            raise RuntimeError("forward() returned %d during capture" % rc)

    def forward_same_layer(st):
        if op.forward(st) != 0:
            raise RuntimeError("forward() failed during capture")

    layer_replays = kernel_replays = prefill_replays = same_layer_replays = same_kernel_replays = None
    if not args.eager:
        # The K layer calls recorded once into a HIP graph and replayed: the way a serving loop runs a decode step
        # (all layers in one graph).  Every kernel runs on every replay; the replays follow each other without a
        # host synchronisation, so the chip is in its sustained state for all but the first.
        try:
            layer_replays = replay_times(forward_on)
            step_s = float(np.median(layer_replays)) * 1e-6
            launch = "HIP graph of %d layer calls, %d replays back to back, median replay" % (args.steps, replays)
            kernel_replays = replay_times(lambda st: dev.decode_only(num_token_ranges=plan.num_token_ranges, workspace=ws,
                                                                      stage=1, stream=st, layer_idx=next_layer()))
            if n_layers > 1 and not args.no_same_layer:  # the regime in which every call re-reads the same layer, for comparison
                same_layer_replays = replay_times(forward_same_layer)
                same_kernel_replays = replay_times(lambda st: dev.decode_only(num_token_ranges=plan.num_token_ranges,
                                                                               workspace=ws, stage=1, stream=st, layer_idx=0))
            if bt.batch > bt.decoding_batches:
                def prefill_on(st):
                    if layer_ops[next_layer()].forward_prefill(st) != 0:
                        raise RuntimeError("forward_prefill() failed during capture")
                prefill_replays = replay_times(prefill_on)
        except Exception as exc:  # the eager timing above stands
            torch.cuda.synchronize()
            launch = "one launch per kernel from the host (graph capture failed: %s)" % str(exc)[:160]

    # per-kernel durations of an event-separated launch loop: an event record between two launches
    def time_stage(fn, n):
        fn()
        torch.cuda.synchronize()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
        for a, b in evs:
            a.record(stream)
            fn()
            b.record(stream)
        torch.cuda.synchronize()
        ts = sorted(a.elapsed_time(b) * 1e3 for a, b in evs)
        return {"avg_us": float(np.mean(ts)), "median_us": float(ts[len(ts) // 2]), "min_us": float(ts[0])}

    n_ev = max(20, args.steps)
    t_ranges = time_stage(lambda: dev.decode_only(num_token_ranges=plan.num_token_ranges, workspace=ws, stage=1,
                                                  layer_idx=next_layer()), n_ev)
    t_combine = time_stage(lambda: dev.decode_only(num_token_ranges=plan.num_token_ranges, workspace=ws, stage=2), n_ev)
    t_append = time_stage(lambda: layer_ops[next_layer()].forward_kvstore(stream), n_ev)
    stages = {"decode_ranges": t_ranges, "decode_combine": t_combine, "append": t_append}
    if bt.batch > bt.decoding_batches:
        stages["prefill"] = time_stage(lambda: layer_ops[next_layer()].forward_prefill(stream), n_ev)

    # the projection behind the attention (single-rank row_parallel_linear) on this step's decode rows: a square
    # weight of (heads * head_dim)^2 halves, streamed once per call
    hidden = bt.num_heads * bt.head_dim
    w_proj = (torch.randn((hidden, hidden), device="cuda") * hidden ** -0.5).to(torch.float16)
    proj_in = dev.output[:bt.decoding_batches]
    proj_out = torch.empty((bt.decoding_batches, hidden), dtype=torch.float16, device="cuda")
    proj_ws_bytes = ops.row_parallel_linear_workspace_size(bt.decoding_batches, hidden, hidden)
    proj_ws = torch.empty(proj_ws_bytes, dtype=torch.uint8, device="cuda") if proj_ws_bytes else None
    stages["o_proj"] = time_stage(lambda: ops.row_parallel_linear(proj_in, w_proj, None, proj_out, workspace=proj_ws), n_ev)
    proj_replays = None
    if not args.eager:
        try:
            proj_replays = replay_times(lambda st: ops.row_parallel_linear(proj_in, w_proj, None, proj_out, workspace=proj_ws, stream=st))
        except Exception:
            torch.cuda.synchronize()

    if args.calibration_copy_mib:
        src = torch.ones(args.calibration_copy_mib << 20, dtype=torch.int8, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    dec_bytes = bt.decode_algorithmic_bytes()
    kernel_name = dev.decode_only(num_token_ranges=plan.num_token_ranges, workspace=ws, name_only=True)
    # the dominant kernel's launch duration: back to back where the graph could be built, else the launch loop
    kernel_us = float(np.mean(kernel_replays)) if kernel_replays else t_ranges["avg_us"]
    achieved = dec_bytes / (kernel_us * 1e-6) / 1e9
    out = {
        "metric": "int8-KV decode attention: achieved HBM GB/s over the whole layer call (us/layer in us_per_layer)",
        "value": dec_bytes / step_s / 1e9,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": step_s * 1e3,
        "us_per_layer": step_s * 1e6,
        "us_per_layer_eager": eager_s * 1e6,
        "us_per_layer_eager_from_idle": eager_from_idle_s * 1e6,
        "launch": launch,
        "replays_us_per_layer": summary(layer_replays) if layer_replays else None,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 cache, fp16 in/out, fp32 accumulate",
        "data": "synthetic (numpy default_rng(%d); cache filled through the HIP quantise/append kernel)" % bt.seed,
        "config": {
            "workload": "%s: %d decode seqs, %d q / %d kv heads, D=%d, %d kv tokens (max %d), cache_mode %d%s; %s" % (
                bt.name, bt.decoding_batches, bt.num_heads, bt.num_kv_heads, bt.head_dim, bt.decode_kv_tokens,
                bt.max_kvlen, bt.cache_mode,
                ", + %d prefill seqs (%d query rows)" % (bt.batch - bt.decoding_batches,
                                                         int(bt.q_lens[bt.decoding_batches:].sum()))
                if bt.batch > bt.decoding_batches else "",
                "call i on layer i mod %d of a %.1f GB cache (%s)" % (
                    n_layers, (dev.cache.numel() + 2 * dev.scale.numel()) / 1e9, bt.layout.kind)
                if n_layers > 1 else "every call on the one layer of the cache (%s)" % bt.layout.kind),
            "layers": n_layers,
            "cache_layout": bt.layout.kind,
            "algorithmic_bytes": dec_bytes,
            "token_ranges": int(plan.num_token_ranges),
            "kv_heads_per_group": int(plan.kv_heads_per_group),
            "q_heads_per_pass": int(plan.q_heads_per_pass),
            "step": "append + decode (token-range kernel + combine)" + (" + prefill" if "prefill" in stages else "") +
                    (", decode on a second stream beside the prefill" if args.two_streams and "prefill" in stages else ""),
        },
        "stages_us": stages,
        "roofline": {
            "kernel": kernel_name,
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": read_traffic(bt.name, kernel_name),
            "traffic_source": "profiles/decode_attention_%s_traffic.txt (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE: "
                              "recorded in runs of their own, not by this process)" % bt.name,
            "kernel_us": kernel_us,
            "kernel_us_regime": ("mean over %d back-to-back replays of a graph of %d launches of this kernel"
                                 % (replays, args.steps)) if kernel_replays else "event-separated launch loop",
            "kernel_us_replays": summary(kernel_replays) if kernel_replays else None,
            "kernel_us_launch_loop": t_ranges["avg_us"],
            "frac_launch_loop": dec_bytes / (t_ranges["avg_us"] * 1e-6) / 1e9 / HBM_PEAK_GBS,
        },
    }
    if same_layer_replays:
        same_us = float(np.median(same_layer_replays))
        same_k = float(np.mean(same_kernel_replays))
        out["same_layer"] = {"note": "every call on layer 0 (a re-read of the same bytes may hit the memory-side cache); "
                                     "not the headline", "us_per_layer": same_us, "value": dec_bytes / same_us / 1e3,
                             "kernel_us": same_k, "kernel_frac": dec_bytes / same_k / 1e3 / HBM_PEAK_GBS}
    proj_us = float(np.mean(proj_replays)) if proj_replays else stages["o_proj"]["avg_us"]
    proj_bytes = hidden * hidden * 2
    out["o_proj"] = {"kernel": "wavek_linear_kernel + linear_reduce_kernel" if proj_ws_bytes else "wavek_linear_kernel", "rows": int(bt.decoding_batches), "in_features": hidden,
                     "out_features": hidden, "bound": "hbm", "weight_bytes": proj_bytes, "kernel_us": proj_us,
                     "achieved": proj_bytes / (proj_us * 1e-6) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": proj_bytes / (proj_us * 1e-6) / 1e9 / HBM_PEAK_GBS,
                     "kernel_us_launch_loop": stages["o_proj"]["avg_us"],
                     "note": "not part of `value`: the step after the layer call, timed on its own"}
    if "prefill" in stages:
        fl = bt.prefill_flops()
        pf_us = float(np.mean(prefill_replays)) if prefill_replays else stages["prefill"]["avg_us"]
        out["prefill"] = {"flops": fl, "kernel_us": pf_us, "achieved_tflops": fl / (pf_us * 1e-6) / 1e12,
                          "peak_tflops": 2500.0, "frac": fl / (pf_us * 1e-6) / 1e12 / 2500.0,
                          "kernel_us_replays": summary(prefill_replays) if prefill_replays else None,
                          "kernel_us_launch_loop": stages["prefill"]["avg_us"]}
    if args.extras and not args.eager:
        out["extras"] = extras(torch, ops, dev, bt, replay_times)
    if not args.no_cpu_baseline:
        oracle = entry.load_oracle()
        # layer 0 as a cache of one layer in the same order of axes
        lay, lay1 = bt.layout, wl.CacheLayout(1, bt.layout.pool_tokens, bt.num_kv_heads, bt.head_dim, bt.layout.kind)
        cache0 = torch.empty(lay1.cache_shape(), dtype=torch.int8, device=dev.device)
        scale0 = torch.empty(lay1.scale_shape(), dtype=torch.float16, device=dev.device)
        lay1.canonical(cache0)[0].copy_(lay.canonical(dev.cache)[0])
        lay1.canonical(scale0)[0].copy_(lay.canonical(dev.scale)[0])
        out["cpu_baseline"] = cpu_baseline(oracle, bt, lay1, q, k, v, cache0.cpu().numpy(), scale0.cpu().numpy())
    print(json.dumps(out))


if __name__ == "__main__":
    main()
