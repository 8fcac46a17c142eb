#!/usr/bin/env python3
"""Benchmark of the TokenSelect decode hot path on one MI355X.

A step is one layer of the patched decode forward after the KV store
(fingerprint -> score -> soft vote -> top-k -> index assembly -> sparse decode
attention) over one synthetic batch resident in HBM, issued as a single
``ts_decode_layer`` call.  The default workload is the Llama-3-8B layer at
128K context in a page-16 KV pool (``--workload c2``); ``c1``, ``c3`` and
``c5`` are the other layer shapes, ``c4`` the 64-step selection-cache trace
(there a step also stores the new token's K/V and consults the cache),
``prefill`` one 512-row chunk of the extend forward on top of a 128K context,
``model`` the whole 32-layer Llama-3-8B-shaped decoder (batch 4, 256K context per
request, 128 greedy decode steps; there a step is one decode step and the value is
tokens/s).

Every step reads a different copy of the K/V pool (``--pools``, default 4, as
consecutive layers of a model do): the copies together exceed the 256 MB
last-level cache, so the keys really stream from HBM in every timed pass.

Prints one JSON line: the per-layer latency, the roofline figures of the
dominant kernel (algorithmic bytes / HIP-event time of the call that streams the
keys: ``ts_select``, the whole selection in one kernel, when the batch fits it,
else ``ts_score``), the same for the stand-alone scoring kernel and the gather
attention, and the CPU oracle timed on the host cores.  The default run appends a
compact line for each of the other workloads, every one measured by a child process
of this script, started before this process touches the GPU (``--no-extra`` leaves
them out, ``--extra-in-process`` measures them here).
"""

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

# HBM bytes per launch of the dominant kernel, from `rocprofv3 --pmc FETCH_SIZE` and
# `--pmc WRITE_SIZE` runs of this script (KiB per dispatch, scaled by what the same
# counters read for the 256 MiB copy of --calibration-copy); the runs and their
# figures are recorded under profiles/.  Workloads not measured that way give null.
# Each figure carries the commit of the kernels it was measured on: a later change to the
# kernel makes it stale until the two counter runs are repeated.
MEASURED_TRAFFIC = {  # workload -> (bytes per launch of its dominant kernel, commit); profiles/decode_layer_hbm_traffic.txt
    "C2": (269799462, "e5a4a17"),        # ts_select, score_kernel<8,4,false,2>
    "C3": (2229654966, "e5a4a17"),       # the votes-only launch, score_kernel<8,4,false,3>
    "C5-layer": (2154403375, "e5a4a17"),  # likewise
    "MODEL": (2158824315, "e5a4a17"),     # likewise, inside the 32-layer decoder (page 1)
}
# attn_kernel<4>, same runs
MEASURED_ATTN_TRAFFIC = {"C2": 12261315, "C3": 180831151, "C5-layer": 82185305}


def event_time_us(fn, launches: int, warmup: int, before=None, burst: int = 1):
    """Average duration of `fn(i)`'s work on the current stream, by HIP events
    (torch.cuda.Event records on the stream the library launches on).  A timed span
    holds `burst` back-to-back calls and is divided by it: a pair of events around a
    single short kernel adds several microseconds that are not the kernel's.
    `before()` runs ahead of each start event, outside the timed span."""
    spans, warm_spans = max(launches // burst, 4), max(warmup // burst, 1)
    for i in range(warm_spans):
        if before:
            before()
        for j in range(burst):
            fn(i * burst + j)
    torch.cuda.synchronize()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
             for _ in range(spans)]
    for i, (start, end) in enumerate(pairs):
        if before:
            before()
        start.record()
        for j in range(burst):
            fn(i * burst + j)
        end.record()
    torch.cuda.synchronize()
    times = [s.elapsed_time(e) * 1e3 / burst for s, e in pairs]
    return sum(times) / len(times), min(times)


def cpu_baseline(wl, reps: int, requests=None):
    """The CPU oracle (a restatement of the reference's PyTorch path) on the host
    cores, same inputs as the GPU run; `requests` restricts it to a bounded sample
    of the batch."""
    import oracle
    c = wl.cfg
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    torch.set_num_threads(threads)
    idx = list(range(len(wl.seq_lens))) if requests is None else list(requests)
    H, D = c.num_heads, c.head_dim
    q = wl.q.view(len(wl.seq_lens), H * D)[idx].cpu()
    kp, vp, table = wl.k_pool.cpu(), wl.v_pool.cpu(), wl.table.cpu()
    lens = [wl.seq_lens[b] for b in idx]
    ks = [wl.k_list[b] for b in idx]
    tabs = [oracle.select.expand_page_table(table[b], wl.seq_lens[b], c.page_size) for b in idx]
    sm = c.sm_scale if c.sm_scale is not None else c.head_dim ** -0.5

    def run():
        return oracle.layer.decode_layer(q, kp, vp, tabs, lens, H, D, c.n_init, c.n_local, ks,
                                         c.rope_theta, c.rope_scale, sm, c.logit_cap, c.rope_mode,
                                         c.pool_kernel)

    run()
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        sels, out = run()
        times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2] * 1e6, torch.get_num_threads(), sels, out


def kernel_rooflines(ops, wl, k_pools, v_pools, layer, steps, warmup):
    """HIP-event timings of the calls that move the bytes: the selection (or the
    scoring kernel where the selection does not fit one launch), the stand-alone
    scoring kernel, and the gather attention."""
    c, bt, B = wl.cfg, wl.batch, len(wl.seq_lens)
    dev = wl.q.device
    n_pools = len(k_pools)
    cos, sin = ops.scoring_cos_sin(c.head_dim, c.rope_theta, c.rope_scale, c.n_local, dev)
    qf = ops.rope_apply(wl.q.view(B, c.num_heads, c.head_dim), cos, sin, None)
    score_bytes, attn_bytes = wl.score_bytes(), wl.attn_bytes()

    bufs = ops.score(c, bt, qf, wl.k_pool)
    score_us, score_min = event_time_us(
        lambda i: ops.score(c, bt, qf, k_pools[i % n_pools], out=bufs), steps, warmup, burst=8)
    score_only = {"kernel": "ts::score_kernel<Hkv,G,false,1> (ts_score: scores written tile-major)",
                  "achieved": round(score_bytes / score_us / 1e3, 1), "peak": HBM_PEAK_GBS,
                  "unit": "GB/s", "frac": round(score_bytes / score_us / 1e3 / HBM_PEAK_GBS, 4),
                  "bytes_per_launch": score_bytes, "us_per_launch": round(score_us, 2),
                  "us_min": round(score_min, 2)}
    del bufs

    if ops.select_supported(c, B, bt.max_seq_len):
        # The selection kernel alone: ts_select's small clearing kernel (inside
        # ts_decode_layer the rotation kernel does that job) runs ahead of the timed
        # span, on one workspace per launch of a burst, and a span is a burst of
        # back-to-back launches, so that the figure is the kernel's duration as a kernel
        # trace shows it rather than that plus the cost of a pair of events.
        burst = 8
        spaces = [ops.select_workspace(c, bt, dev) for _ in range(burst)]

        def clear_all():
            for space in spaces:
                ops.select_clear(c, bt, space)

        def run_select(i):
            ops.select(c, bt, qf, k_pools[i % n_pools], workspace=spaces[i % burst], cleared=True)

        dom_us, dom_min = event_time_us(run_select, steps, warmup, before=clear_all, burst=burst)
        if any(ops.select_fault(c, bt, space) for space in spaces):
            sys.exit("bench.py: a grid-wide wait of the selection kernel gave up")
        dom_kernel = "ts::score_kernel<Hkv,G,false,2> (ts_select: score + vote + top-k in one launch)"
    elif ops.layer_selection_form(c, bt) == 1:
        # Scores and votes request by request, the scores never in memory: the fused kernel
        # in its votes-only form (+ one small clearing kernel), one launch whose phases are
        # packed by the host's lengths, or by max_seq_len without them; the figure is the
        # bytes of all requests over the launch's time.
        space = ops.select_workspace(c, bt, dev)
        dom_us, dom_min = event_time_us(
            lambda i: ops.score_vote(c, bt, qf, k_pools[i % n_pools], workspace=space), steps, warmup,
            burst=4)
        dom_kernel = ("ts::score_kernel<Hkv,G,false,3> votes-only form, one launch whose phases are packed "
                      + ("by the host's lengths" if bt.host_seq_lens is not None else "by max_seq_len")
                      + " (ts_score_vote: score + statistics + vote)")
    else:
        dom_us, dom_min, dom_kernel = score_us, score_min, score_only["kernel"]
    gbs = score_bytes / dom_us / 1e3
    roofline = {"bound": "hbm", "kernel": dom_kernel, "achieved": round(gbs, 1),
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                "traffic": MEASURED_TRAFFIC.get(wl.name.split()[0], (None, None))[0],
                "traffic_measured_at": MEASURED_TRAFFIC.get(wl.name.split()[0], (None, None))[1],
                "bytes_per_launch": score_bytes, "us_per_launch": round(dom_us, 2),
                "us_min": round(dom_min, 2)}

    sel, sel_len = layer.sel, layer.sel_len
    attn_us, _ = event_time_us(
        lambda i: ops.sparse_decode_attention(c, wl.q, k_pools[i % n_pools], v_pools[i % n_pools],
                                              sel, sel_len), steps, warmup, burst=8)
    attn = {"kernel": "ts::attn_kernel<G> (+ a 1 us ticket-clearing kernel when called on its own)",
            "achieved": round(attn_bytes / attn_us / 1e3, 1), "unit": "GB/s",
            "frac": round(attn_bytes / attn_us / 1e3 / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_ATTN_TRAFFIC.get(wl.name.split()[0]),
            "bytes_per_launch": attn_bytes, "us_per_launch": round(attn_us, 2)}
    return roofline, score_only, attn


def bench_layer(args, ops, workloads, dev, which=None):
    make = {"c1": workloads.config1, "c2": workloads.config2, "c3": workloads.config3,
            "c5": workloads.config5_layer}[which or args.workload]
    wl = make(dev)
    # Batches too large for one ts_select launch: the lengths are handed over on the host as
    # well (a serving framework holds them there), so that the scoring is one launch whose
    # phases are packed by what the requests hold.
    wl.host_lengths = (which or args.workload) in ("c3", "c5") and not args.device_lengths_only
    c, B = wl.cfg, len(wl.seq_lens)
    if not args.no_hint:
        # Where the k-th vote lay at the layer's previous step, kept by the caller per (request,
        # layer) as a serving stack would: the steps of this benchmark repeat one decode step,
        # so the guess is always right here; --no-hint measures the selection without it.
        wl.hint = torch.zeros(B, dtype=torch.int32, device=dev)
    bt = wl.batch
    layer = ops.DecodeLayer(c, B, bt.max_seq_len, dev)
    n_pools = max(1, args.pools)
    k_pools = [wl.k_pool] + [wl.k_pool.clone() for _ in range(n_pools - 1)]
    v_pools = [wl.v_pool] + [wl.v_pool.clone() for _ in range(n_pools - 1)]

    def step(i):
        layer(wl.q, k_pools[i % n_pools], v_pools[i % n_pools], bt)

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    us_per_layer = (time.perf_counter() - t0) / args.steps * 1e6

    roofline, score_only, attn = kernel_rooflines(ops, wl, k_pools, v_pools, layer, args.steps,
                                                  args.warmup)
    if args.calibration_copy:  # a plain copy of known size for the counter runs
        src = torch.empty((256 << 20,), dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()

    result = {
        "metric": "us_per_layer_decode (score+top-k+sparse attn)",
        "value": round(us_per_layer, 2), "unit": "us", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(us_per_layer / 1e3, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": wl.name, "batch": B, "seq_lens_max": max(wl.seq_lens),
                   "page_size": c.page_size, "top_k": c.top_k, "n_init": c.n_init,
                   "n_local": c.n_local, "kv_pool_copies": n_pools,
                   "lengths_on_host_too": bool(wl.host_lengths),
                   "threshold_hint": not args.no_hint,
                   "selection": {2: "ts_select", 1: "ts_score_vote + top-k kernels",
                                 0: "ts_score + ts_vote + top-k kernels"}[ops.layer_selection_form(c, bt)]},
        "tokens_per_s": round(B / (us_per_layer * 1e-6 * args.layers), 1),
        "tokens_per_s_note": f"selection+attention only, {args.layers} layers per token",
        "roofline": roofline, "score_only": score_only, "gather_attention": attn,
    }

    if not args.no_cpu_baseline:
        # Bounded sample: the whole batch where that is a few hundred ms of CPU work,
        # else its first two requests.
        sample = None if sum(wl.seq_lens) <= 300000 else [0, 1][:args.cpu_requests]
        cpu_us, cores, ref_sels, ref_out = cpu_baseline(wl, args.cpu_reps, sample)
        what = f"the full {wl.name} layer" if sample is None else \
            f"requests {sample} (L={[wl.seq_lens[b] for b in sample]}) of {wl.name}"
        result["cpu_baseline"] = {
            "value": round(cpu_us, 1), "unit": "us", "cores": cores, "kind": "port",
            "sample": f"{what}, median of {args.cpu_reps} repetitions after one warm-up "
                      "(PyTorch CPU oracle)"}
        # Parity of this very run against the oracle.
        idx = list(range(B)) if sample is None else sample
        S = [int(x) for x in layer.sel_len.tolist()]
        same = all(torch.equal(layer.sel[b, :S[b]].cpu(), ref_sels[i]) for i, b in enumerate(idx))
        err = (layer.out[idx].cpu().float() - ref_out.float()).abs().max().item()
        result["parity"] = {"selected_slots_identical": bool(same),
                            "attn_max_abs_err": round(err, 5)}
    return result


def bench_trace(args, ops, workloads, dev):
    """Selection-cache trace: `trace_steps` consecutive decode steps of one layer, the
    new token's K/V stored first, AR(1) queries with occasional jumps, cosine reuse
    threshold bf16(0.9).  Reports the amortised time per step and the hit rate."""
    steps = args.trace_steps
    ps = args.page_size
    wl = workloads.config4(dev, steps=steps, page_size=ps)
    c, B = wl.cfg, len(wl.seq_lens)
    L0 = wl.seq_lens[0]
    qs = workloads.ar1_queries(B, c.num_heads * c.head_dim, steps, dev)
    gen = torch.Generator(device=dev).manual_seed(7)
    k_new = torch.randn((steps, B, c.num_kv_heads * c.head_dim), generator=gen, device=dev).bfloat16()
    v_new = torch.randn((steps, B, c.num_kv_heads * c.head_dim), generator=gen, device=dev).bfloat16()
    # New tokens go to the slots a serving framework would hand over (per-token table),
    # or, with pages, to fresh pages the store kernel takes from the device-side free list.
    free = wl.free_pages[:B * steps].view(steps, B) if ps == 1 else None
    table0 = torch.zeros((B, -(-(L0 + steps) // ps)), dtype=torch.int32, device=dev)
    table0[:, :wl.table.shape[1]] = wl.table
    layer = ops.DecodeLayer(c, B, L0 + steps, dev)

    def run_trace():
        table, seq = table0.clone(), wl.seq_lens_dev.clone()
        cache = ops.SelectionCache.allocate(c, B, dev)
        hint = None if args.no_hint else torch.zeros(B, dtype=torch.int32, device=dev)
        pages = ops.PagePool.of(wl.free_pages) if ps > 1 else None
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for t in range(steps):
            # store + layer in one call, as the reference's decode forward does both
            layer.step(qs[t], k_new[t], v_new[t], None if pages else free[t], wl.k_pool, wl.v_pool,
                       ops.Batch(seq, table, L0 + t + 1, hint=hint), cache, pages=pages)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e6, cache

    for _ in range(max(1, args.warmup // steps)):
        run_trace()
    reps = max(1, args.steps // steps)
    runs = [run_trace() for _ in range(reps)]
    us_per_step = sum(r[0] for r in runs) / reps
    counters = runs[-1][1].counters.cpu()
    hits, lookups = int(counters[:, 0].sum()), int(counters[:, 1].sum())

    result = {
        "metric": "us_per_layer_decode (selection-cache trace: kv store + cache + select + attn)",
        "value": round(us_per_step, 2), "unit": "us", "n_gpus": 1, "steps": reps * steps,
        "warmup": max(1, args.warmup // steps) * steps, "ms_per_step": round(us_per_step / 1e3, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": wl.name, "batch": B, "seq_lens_max": L0 + steps, "page_size": ps,
                   "top_k": c.top_k, "n_init": c.n_init, "n_local": c.n_local,
                   "trace_steps": steps, "ar1_rho": 0.95, "jump_p": 0.1,
                   "threshold": runs[-1][1].threshold, "kv_pool_copies": 1},
        "hit_rate": round(hits / max(lookups, 1), 4), "hits": hits, "lookups": lookups,
        "tokens_per_s": round(B / (us_per_step * 1e-6 * args.layers), 1),
        "tokens_per_s_note": f"selection+attention only, {args.layers} layers per token",
        "cpu_baseline": None,
    }
    # What a step needs from HBM: the keys of the requests that missed (a hit scores nothing)
    # and the gathered K/V rows of every request, over the whole step's time (the store, the
    # cache comparison, the selection and the attention): a figure for the trace as a whole,
    # not for one kernel.
    row = c.num_kv_heads * c.head_dim * 2
    miss_bytes = (lookups - hits) * ((L0 + steps // 2 - c.n_init - c.n_local) * row)
    gather_bytes = lookups * c.max_sel * 2 * row
    step_bytes = (miss_bytes + gather_bytes) / steps
    gbs = step_bytes / us_per_step / 1e3
    result["roofline"] = {"bound": "hbm", "kernel": "whole step (ts_kv_store + ts_decode_layer with the cache)",
                          "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                          "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                          "bytes_per_step": int(step_bytes), "us_per_step": round(us_per_step, 2)}
    return result


MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 matrix peak


def bench_prefill(args, ops, workloads, dev):
    """One chunk of the patched extend forward on top of a 128K context: store the
    chunk's K/V, fingerprint of the chunk, selection, causal sparse attention of the
    chunk's 512 rows.  Each step serves a different copy of the pool."""
    L0, m = args.prefill_context, args.prefill_rows
    wl = workloads.build("PREFILL llama3-8b L%d chunk%d k2048 page1" % (L0, m), workloads.LLAMA3_8B,
                         [L0], [2048], 1, dev, seed=5, extra_pages=m)
    c = wl.cfg
    gen = torch.Generator(device=dev).manual_seed(6)
    q = torch.randn((m, c.num_heads * c.head_dim), generator=gen, device=dev).bfloat16()
    k_new = torch.randn((m, c.num_kv_heads, c.head_dim), generator=gen, device=dev).bfloat16()
    v_new = torch.randn((m, c.num_kv_heads, c.head_dim), generator=gen, device=dev).bfloat16()
    loc = torch.arange(L0, L0 + m, dtype=torch.int32, device=dev)
    table0 = torch.zeros((1, L0 + m), dtype=torch.int32, device=dev)
    table0[0, :L0] = wl.table[0, :L0]
    n_pools = max(1, args.pools)
    k_pools = [wl.k_pool] + [wl.k_pool.clone() for _ in range(n_pools - 1)]
    v_pools = [wl.v_pool] + [wl.v_pool.clone() for _ in range(n_pools - 1)]
    layer = ops.PrefillChunk(c, L0 + m, dev, max_rows=m)
    tables = [table0.clone() for _ in range(n_pools)]
    seqs = [wl.seq_lens_dev.clone() for _ in range(n_pools)]

    def step(i):
        p = i % n_pools
        seqs[p].fill_(L0)          # the chunk is appended afresh every time
        # store + chunk in one call, as the reference's extend forward has them per chunk
        return layer.step(q, k_new, v_new, loc, k_pools[p], v_pools[p], ops.Batch(seqs[p], tables[p], L0 + m))

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    us_per_chunk = (time.perf_counter() - t0) / args.steps * 1e6

    out, sel, _, sel_len = step(0)
    torch.cuda.synchronize()
    S = int(sel_len[0])
    sel0 = sel[0].contiguous()
    attn_us, attn_min = event_time_us(
        lambda i: ops.sparse_prefill_attention(c, q, k_pools[i % n_pools], v_pools[i % n_pools], sel0,
                                               sel_len, c.max_sel), args.steps, args.warmup, burst=8)
    visible = sum(S - m + i + 1 for i in range(m))                 # (row, key) pairs under the mask
    flops = 4 * c.num_heads * c.head_dim * visible                 # QK^T and PV, 2 flops per MAC
    tflops = flops / attn_us / 1e6
    result = {
        "metric": "us_per_layer_prefill_chunk (kv store+fingerprint+select+causal sparse attn)",
        "value": round(us_per_chunk, 2), "unit": "us", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(us_per_chunk / 1e3, 5),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": wl.name, "batch": 1, "seq_lens_max": L0 + m, "chunk_rows": m,
                   "page_size": 1, "top_k": c.top_k, "n_init": c.n_init, "n_local": c.n_local,
                   "kv_pool_copies": n_pools},
        "prompt_tokens_per_s": round(m / (us_per_chunk * 1e-6 * args.layers), 1),
        "tokens_per_s_note": f"selection+attention only, {args.layers} layers per token",
        "roofline": {"bound": "mfma", "kernel": "ts::prefill_attn_kernel<G> (+ the 7 us gather pass)",
                     "achieved": round(tflops, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "flops_per_launch": flops, "us_per_launch": round(attn_us, 2),
                     "us_min": round(attn_min, 2)},
    }
    if not args.no_cpu_baseline:
        import oracle
        torch.set_num_threads(int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
        kc, vc, tab = k_pools[0].cpu(), v_pools[0].cpu(), tables[0][0].cpu()
        qc = q.cpu()
        qf = ops.fingerprint(c, q.view(m, c.num_heads, c.head_dim), layer.cos, layer.sin).cpu()
        sm = c.head_dim ** -0.5

        def run():
            return oracle.prefill.prefill_chunk(qc, kc, vc, tab, L0 + m, c.num_heads, c.head_dim,
                                                c.n_init, c.n_local, c.top_k, c.rope_theta,
                                                c.rope_scale, sm, qf_override=qf)

        run()
        times = []
        for _ in range(args.cpu_reps):
            t0 = time.perf_counter()
            ref_slots, ref_out = run()
            times.append(time.perf_counter() - t0)
        times.sort()
        result["cpu_baseline"] = {
            "value": round(times[len(times) // 2] * 1e6, 1), "unit": "us",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"the chunk's selection + attention (no KV store), median of {args.cpu_reps} "
                      "repetitions after one warm-up (PyTorch CPU oracle)"}
        same = torch.equal(sel[0, :S].cpu(), ref_slots)
        err = (out.cpu().float() - ref_out.float()).abs().max().item()
        result["parity"] = {"selected_slots_identical": bool(same),
                            "attn_max_abs_err": round(err, 5)}
    return result


def bench_model(args, ops, dev):
    """The full-model configuration: a random-initialised Llama-3-8B-shaped decoder
    (bf16 weights N(0, 0.02)), `model_batch` requests with `model_context` prefilled
    random KV tokens each, TokenSelect on all layers, greedy decoding.  A step is
    one decode step of the whole batch through all layers."""
    from tokenselect_amd.model import Decoder, ModelConfig
    mc = ModelConfig(layers=args.layers, top_k=args.model_top_k)
    B, L = args.model_batch, args.model_context
    t0 = time.perf_counter()
    m = Decoder(mc, [L] * B, args.warmup + args.steps + 1, dev, seed=4)
    torch.cuda.synchronize()
    build_s = time.perf_counter() - t0
    c = m.cfg
    tokens = torch.arange(1, B + 1, device=dev)
    tokens = m.generate(tokens, args.warmup)[-1] if args.warmup else tokens
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    tokens = m.generate(tokens, args.steps)[-1]
    torch.cuda.synchronize()
    step_s = (time.perf_counter() - t0) / args.steps

    # One more step, traced, for the parity check and the kernel timings.
    trace = []
    m.decode_step(tokens, trace)
    torch.cuda.synchronize()
    Lnow = L + args.warmup + args.steps + 1
    bt = ops.Batch(m.num_tokens[0], m.table, Lnow,
                   host_seq_lens=torch.full((B,), Lnow, dtype=torch.int32))  # as the model's layers pass them
    row = c.num_kv_heads * c.head_dim * 2
    score_bytes = B * ((Lnow - c.n_init - c.n_local) * row + Lnow * 4 + c.num_heads * c.head_dim * 2)
    cos, sin = ops.scoring_cos_sin(c.head_dim, c.rope_theta, c.rope_scale, c.n_local, dev)
    qf = ops.rope_apply(trace[0][0].view(B, c.num_heads, c.head_dim), cos, sin, None)
    bufs = ops.score(c, bt, qf, m.k_pools[0])
    score_us, score_min = event_time_us(
        lambda i: ops.score(c, bt, qf, m.k_pools[i % mc.layers], out=bufs), 2 * mc.layers, mc.layers,
        burst=4)
    del bufs
    score_only = {"kernel": "ts::score_kernel<Hkv,G,false,1> (ts_score, stand-alone)",
                  "achieved": round(score_bytes / score_us / 1e3, 1), "unit": "GB/s",
                  "frac": round(score_bytes / score_us / 1e3 / HBM_PEAK_GBS, 4),
                  "us_per_launch": round(score_us, 2), "us_min": round(score_min, 2)}
    dom_kernel = "ts::score_kernel<Hkv,G,false,1> (ts_score, one launch per layer)"
    if ops.layer_selection_form(c, bt) == 1:
        # What the layers of this model run: scores and votes request by request, the scores
        # never in memory (the requests as phases of one launch; the figure is all their
        # bytes over all its time).
        space = ops.select_workspace(c, bt, dev)
        score_us, score_min = event_time_us(
            lambda i: ops.score_vote(c, bt, qf, m.k_pools[i % mc.layers], workspace=space),
            2 * mc.layers, mc.layers, burst=4)
        dom_kernel = (f"ts::score_kernel<Hkv,G,false,3> votes-only form, {B} requests as phases of one "
                      "launch per layer (ts_score_vote: score + statistics + vote)")
        del space
    gbs = score_bytes / score_us / 1e3
    weights = sum(w.numel() * 2 for ws in (m.wqkv, m.wo, m.w_gate_up, m.w_down) for w in ws) \
        + m.lm_head.numel() * 2
    sel_rows = B * c.max_sel
    step_bytes = weights + mc.layers * (score_bytes + sel_rows * (2 * row + 4))
    result = {
        "metric": "decode tokens/s, full model (all layers TokenSelect, greedy)",
        "value": round(B / step_s, 2), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "C5 llama3-8b-shaped decoder B%d L%d k%d page1, %d layers"
                               % (B, L, c.top_k, mc.layers),
                   "batch": B, "seq_lens_max": Lnow, "page_size": 1, "top_k": c.top_k,
                   "n_init": c.n_init, "n_local": c.n_local, "hidden": mc.hidden,
                   "intermediate": mc.intermediate, "vocab": mc.vocab,
                   "weights": "random N(0, 0.02) bf16", "kv": "prefilled random N(0,1) bf16"},
        "us_per_layer": round(step_s * 1e6 / mc.layers, 2),
        "setup_s": round(build_s, 1),
        "hbm_bytes_per_step": step_bytes,
        "hbm_frac_whole_step": round(step_bytes / step_s / 1e9 / HBM_PEAK_GBS, 4),
        "roofline": {"bound": "hbm", "kernel": dom_kernel,
                     "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": MEASURED_TRAFFIC["MODEL"][0] if (B, L, c.top_k) == (4, 262144, 4096) else None,
                     "traffic_measured_at": MEASURED_TRAFFIC["MODEL"][1],
                     "bytes_per_launch": score_bytes, "us_per_launch": round(score_us, 2),
                     "us_min": round(score_min, 2)},
        "score_only": score_only,
    }
    if not args.no_cpu_baseline:
        import oracle
        torch.set_num_threads(int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
        layer_ix = mc.layers - 1
        q, _, _, attn, sel, sel_len = trace[layer_ix]
        kc, vc = m.k_pools[layer_ix].cpu(), m.v_pools[layer_ix].cpu()
        tab = m.table[0].cpu()
        q0 = q[:1].cpu()

        def run():
            return oracle.layer.decode_layer(q0, kc, vc, [tab], [Lnow], c.num_heads, c.head_dim,
                                             c.n_init, c.n_local, [c.top_k], c.rope_theta,
                                             c.rope_scale, c.head_dim ** -0.5)

        run()
        times = []
        for _ in range(args.cpu_reps):
            t0 = time.perf_counter()
            ref_sels, ref_out = run()
            times.append(time.perf_counter() - t0)
        times.sort()
        per_request_layer = times[len(times) // 2]
        result["cpu_baseline"] = {
            "value": round(1.0 / (per_request_layer * mc.layers), 4), "unit": "tokens/s",
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"selection + attention of request 0 on layer {layer_ix} at the last decode "
                      f"step ({per_request_layer * 1e3:.1f} ms, median of {args.cpu_reps} after one "
                      f"warm-up, PyTorch CPU oracle), scaled by {mc.layers} layers per token; the "
                      "projections and the MLP are not in it"}
        S = int(sel_len[0])
        same = torch.equal(sel[0, :S].cpu(), ref_sels[0])
        err = (attn[0].cpu().float() - ref_out[0].float()).abs().max().item()
        result["parity"] = {"selected_slots_identical": bool(same),
                            "attn_max_abs_err": round(err, 5)}
    return result


def _layer_line(r):
    roof = r["roofline"]
    return {"workload": r["config"]["workload"], "us_per_layer": r["value"],
            "dominant_kernel": roof["kernel"].split(" ")[0], "us_per_launch": roof["us_per_launch"],
            "bytes_per_launch": roof["bytes_per_launch"], "frac": roof["frac"],
            "traffic": roof["traffic"], "score_only_frac": r["score_only"]["frac"],
            "attn_us": r["gather_attention"]["us_per_launch"], "parity": r.get("parity")}


def _trace_line(r):
    return {"workload": r["config"]["workload"], "us_per_step": r["value"],
            "hit_rate": r["hit_rate"], "bytes_per_step": r["roofline"]["bytes_per_step"],
            "frac": r["roofline"]["frac"]}


def _prefill_line(r):
    return {"workload": r["config"]["workload"], "us_per_chunk": r["value"],
            "dominant_kernel": "ts::prefill_attn_kernel<G>", "bound": "mfma",
            "us_per_launch": r["roofline"]["us_per_launch"],
            "flops_per_launch": r["roofline"]["flops_per_launch"],
            "tflops": r["roofline"]["achieved"], "frac": r["roofline"]["frac"],
            "parity": r.get("parity")}


def _model_line(r):
    return {"workload": r["config"]["workload"], "tokens_per_s": r["value"],
            "greedy_steps": r["steps"], "ms_per_decode_step": r["ms_per_step"],
            "us_per_layer": r["us_per_layer"], "hbm_frac_whole_step": r["hbm_frac_whole_step"],
            "dominant_kernel": r["roofline"]["kernel"].split(" ")[0],
            "us_per_launch": r["roofline"]["us_per_launch"], "frac": r["roofline"]["frac"],
            "traffic": r["roofline"]["traffic"],
            "cpu_tokens_per_s": (r.get("cpu_baseline") or {}).get("value"),
            "parity": r.get("parity")}


# The other configurations of the default run: fewer steps, the oracle on one request (parity
# only).  (name, arguments of this script, what makes the compact line of the result)
EXTRA = [
    ("c1", ["--workload", "c1", "--steps", "50", "--warmup", "10"], _layer_line),
    ("c3", ["--workload", "c3", "--steps", "50", "--warmup", "10"], _layer_line),
    ("c5", ["--workload", "c5", "--steps", "50", "--warmup", "10"], _layer_line),
    ("c4", ["--workload", "c4", "--steps", "64", "--warmup", "64", "--page-size", "1"], _trace_line),
    ("c4-pages", ["--workload", "c4", "--steps", "64", "--warmup", "64", "--page-size", "16"], _trace_line),
    # one 512-row chunk of the extend forward on a 128K context
    ("prefill", ["--workload", "prefill", "--steps", "50", "--warmup", "10"], _prefill_line),
    # the whole 32-layer decoder (the reference's full-model configuration) over 32 greedy steps
    ("model", ["--workload", "model", "--steps", "32", "--warmup", "2"], _model_line),
]
EXTRA_COMMON = ["--pools", "4", "--cpu-reps", "1", "--cpu-requests", "1", "--no-extra"]


def extra_in_own_processes():
    """Every other workload measured by a child process of this script, one after the other,
    before this process touches the GPU: a process of its own gives a workload the device
    memory as a freshly started server finds it, whatever other workloads allocated and
    freed (in one process C3 and C5 came out up to 3 % slower by that).  Returns the compact
    lines, None where a child could not be had."""
    import subprocess
    lines = []
    for name, argv, line_of in EXTRA:
        t0 = time.perf_counter()
        try:
            res = subprocess.run([sys.executable, os.path.abspath(__file__)] + argv + EXTRA_COMMON,
                                 capture_output=True, text=True, timeout=600)
            if res.returncode != 0:
                raise RuntimeError(f"exit code {res.returncode}: {res.stderr[-400:]}")
            line = line_of(json.loads(res.stdout.strip().splitlines()[-1]))
            line["wall_s"] = round(time.perf_counter() - t0, 1)
            lines.append(line)
        except Exception as e:
            print(f"bench.py: workload {name} in a process of its own: {e}", file=sys.stderr, flush=True)
            lines.append(None)
    return lines


def extra_here(lines, args, ops, workloads, dev):
    """The workloads no child process could be had for, measured in this process."""
    import copy
    import gc
    parser_defaults = copy.copy(args)
    for i, (name, argv, line_of) in enumerate(EXTRA):
        if lines[i] is not None:
            continue
        gc.collect()
        torch.cuda.empty_cache()
        t0 = time.perf_counter()
        small = copy.copy(parser_defaults)
        small.pools, small.cpu_reps, small.cpu_requests = 4, 1, 1
        opts = dict(zip(argv[0::2], argv[1::2]))
        small.steps, small.warmup = int(opts["--steps"]), int(opts["--warmup"])
        small.page_size = int(opts.get("--page-size", 1))
        which = opts["--workload"]
        if which == "c4":
            r = bench_trace(small, ops, workloads, dev)
        elif which == "prefill":
            r = bench_prefill(small, ops, workloads, dev)
        elif which == "model":
            r = bench_model(small, ops, dev)
        else:
            r = bench_layer(small, ops, workloads, dev, which)
        lines[i] = line_of(r)
        lines[i]["wall_s"] = round(time.perf_counter() - t0, 1)
    torch.cuda.empty_cache()
    return lines


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps (default 200; 128 decode steps for the model workload)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps (default 20; model 4)")
    ap.add_argument("--workload", default="c2",
                    choices=["c1", "c2", "c3", "c4", "c5", "prefill", "model"])
    ap.add_argument("--cpu-reps", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--layers", type=int, default=32,
                    help="layers for the tokens/s figure; layers of the model workload")
    ap.add_argument("--model-batch", type=int, default=4)
    ap.add_argument("--model-context", type=int, default=262144)
    ap.add_argument("--model-top-k", type=int, default=4096)
    ap.add_argument("--pools", type=int, default=4,
                    help="copies of the K/V pool cycled through, one per step")
    ap.add_argument("--trace-steps", type=int, default=64, help="decode steps of the c4 trace")
    ap.add_argument("--page-size", type=int, default=1,
                    help="tokens per KV page of the c4 trace (above 1: appends through the page pool)")
    ap.add_argument("--cpu-requests", type=int, default=2,
                    help="requests of a large batch the CPU oracle is run on")
    ap.add_argument("--device-lengths-only", action="store_true",
                    help="c3, c5: do not hand the lengths to the library on the host")
    ap.add_argument("--extra-in-process", action="store_true",
                    help="measure the default run's other workloads in this process, not in child processes")
    ap.add_argument("--no-extra", action="store_true",
                    help="default run: only the headline workload, not the compact lines of the others")
    ap.add_argument("--prefill-context", type=int, default=131072,
                    help="tokens already cached when the measured prefill chunk arrives")
    ap.add_argument("--prefill-rows", type=int, default=512, help="rows of the prefill chunk")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run five 256 MiB device copies (reference for counter runs)")
    ap.add_argument("--no-hint", action="store_true",
                    help="layer workloads: do not hand ts_select the previous step's threshold bin")
    ap.add_argument("--separate-kernels", action="store_true",
                    help="ts_set_fused_select(0): the selection as ts_score + ts_vote + the top-k kernels")
    args = ap.parse_args()
    if args.steps is None:
        args.steps = 128 if args.workload == "model" else 200
    if args.warmup is None:
        args.warmup = 4 if args.workload == "model" else 20
    if args.gpus != 1:
        sys.exit("bench.py: this build measures the one-GPU hot path only; run with --gpus 1 "
                 "(no multi-GPU figure exists for it).")
    extra = None
    if args.workload == "c2" and not args.no_extra and torch.cuda.device_count() > 0:
        # (before this process initialises the GPU)
        extra = [None] * len(EXTRA) if args.extra_in_process else extra_in_own_processes()
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback.")

    from tokenselect_amd import ops, workloads

    dev = torch.device("cuda:0")
    if args.separate_kernels:
        ops.set_fused_select(False)
    if args.workload == "c4":
        result = bench_trace(args, ops, workloads, dev)
    elif args.workload == "prefill":
        result = bench_prefill(args, ops, workloads, dev)
    elif args.workload == "model":
        result = bench_model(args, ops, dev)
    else:
        result = bench_layer(args, ops, workloads, dev)
        if extra is not None:
            result["extra_workloads"] = extra_here(extra, args, ops, workloads, dev)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
