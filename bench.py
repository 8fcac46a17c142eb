#!/usr/bin/env python3
"""Benchmark of the TokenSelect decode hot path on one MI355X.

A step is one layer of the patched decode forward after the KV store
(fingerprint -> score -> soft vote -> top-k -> index assembly -> sparse decode
attention) over one synthetic batch resident in HBM, issued as a single
``ts_decode_layer`` call.  The default workload is the Llama-3-8B layer at
128K context in a page-16 KV pool (``--workload c2``).

Every step reads a different copy of the K/V pool (``--pools``, default 4, as
consecutive layers of a model do): the copies together exceed the 256 MB
last-level cache, so the keys really stream from HBM in every timed pass.

Prints one JSON line: the per-layer latency, the roofline figures of the
scoring kernel (algorithmic bytes / HIP-event time of the call that streams the
keys: ``ts_select``, the whole selection in one kernel, when the batch fits it,
else ``ts_score``) and the CPU oracle timed on the host cores.
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


def event_time_us(fn, launches: int, warmup: int, before=None):
    """Average duration of `fn(i)`'s work on the current stream, HIP events around
    every launch (torch.cuda.Event records on the stream the library launches on).
    `before()` runs ahead of each start event, outside the timed span."""
    for i in range(warmup):
        if before:
            before()
        fn(i)
    torch.cuda.synchronize()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
             for _ in range(launches)]
    for i, (start, end) in enumerate(pairs):
        if before:
            before()
        start.record()
        fn(i)
        end.record()
    torch.cuda.synchronize()
    times = [s.elapsed_time(e) * 1e3 for s, e in pairs]
    return sum(times) / len(times), min(times)


def cpu_baseline(wl, reps: int):
    """The CPU oracle (a restatement of the reference's PyTorch path) on the
    host cores, same inputs as the GPU run."""
    import oracle
    c = wl.cfg
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    torch.set_num_threads(threads)
    q, kp, vp, table = wl.q.cpu(), wl.k_pool.cpu(), wl.v_pool.cpu(), wl.table.cpu()
    tabs = [oracle.select.expand_page_table(table[b], L, c.page_size)
            for b, L in enumerate(wl.seq_lens)]
    sm = c.sm_scale if c.sm_scale is not None else c.head_dim ** -0.5

    def run():
        return oracle.layer.decode_layer(q, kp, vp, tabs, wl.seq_lens, c.num_heads, c.head_dim,
                                         c.n_init, c.n_local, wl.k_list, c.rope_theta, c.rope_scale,
                                         sm, c.logit_cap, c.rope_mode, c.pool_kernel)

    run()
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        sels, out = run()
        times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2] * 1e6, torch.get_num_threads(), sels, out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c2", choices=["c1", "c2", "c3"])
    ap.add_argument("--cpu-reps", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--layers", type=int, default=32, help="layers for the tokens/s figure")
    ap.add_argument("--pools", type=int, default=4,
                    help="copies of the K/V pool cycled through, one per step")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures the one-GPU hot path only; run with --gpus 1 "
                 "(no multi-GPU figure exists for it).")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback.")

    from tokenselect_amd import ops, workloads

    dev = torch.device("cuda:0")
    wl = {"c1": workloads.config1, "c2": workloads.config2, "c3": workloads.config3}[args.workload](dev)
    c, bt, B = wl.cfg, wl.batch, len(wl.seq_lens)
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
    elapsed = time.perf_counter() - t0
    us_per_layer = elapsed / args.steps * 1e6

    # Kernel-level roofline figures: the kernel that streams the keys, and the
    # gather attention.
    cos, sin = ops.scoring_cos_sin(c.head_dim, c.rope_theta, c.rope_scale, c.n_local, dev)
    qf = ops.rope_apply(wl.q.view(B, c.num_heads, c.head_dim), cos, sin, None)
    fused = ops.select_supported(c, B, bt.max_seq_len)
    if fused:
        space = [None]

        def run_select(i):
            space[0] = ops.select(c, bt, qf, k_pools[i % n_pools], workspace=space[0])[4]

        # ts_select = one small clearing kernel + the selection kernel; the clearing
        # kernel (about 2 us) is inside the timed span.
        score_us, score_min = event_time_us(run_select, args.steps, args.warmup)
        if ops.select_fault(c, bt, space[0]):
            sys.exit("bench.py: a grid-wide wait of the selection kernel gave up")
        score_kernel = "ts::score_kernel<Hkv,G,false,2> (ts_select: score + vote + top-k in one launch)"
    else:
        bufs = ops.score(c, bt, qf, wl.k_pool)
        score_us, score_min = event_time_us(
            lambda i: ops.score(c, bt, qf, k_pools[i % n_pools], out=bufs), args.steps, args.warmup)
        score_kernel = "ts::score_kernel<Hkv,G,false,1> (ts_score)"
    sel, sel_len = layer.sel, layer.sel_len
    attn_us, _ = event_time_us(
        lambda i: ops.sparse_decode_attention(c, wl.q, k_pools[i % n_pools], v_pools[i % n_pools],
                                              sel, sel_len),
        args.steps, args.warmup)
    score_bytes, attn_bytes = wl.score_bytes(), wl.attn_bytes()
    score_gbs = score_bytes / score_us / 1e3
    attn_gbs = attn_bytes / attn_us / 1e3

    result = {
        "metric": "us_per_layer_decode (score+top-k+sparse attn)",
        "value": round(us_per_layer, 2),
        "unit": "us",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us_per_layer / 1e3, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": wl.name, "batch": B, "seq_lens_max": max(wl.seq_lens),
                   "page_size": c.page_size, "top_k": c.top_k, "n_init": c.n_init,
                   "n_local": c.n_local, "kv_pool_copies": n_pools},
        "tokens_per_s": round(B / (us_per_layer * 1e-6 * args.layers), 1),
        "tokens_per_s_note": f"selection+attention only, {args.layers} layers per token",
        "roofline": {"bound": "hbm", "kernel": score_kernel, "achieved": round(score_gbs, 1),
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(score_gbs / HBM_PEAK_GBS, 4),
                     "traffic": None, "bytes_per_launch": score_bytes,
                     "us_per_launch": round(score_us, 2), "us_min": round(score_min, 2)},
        "gather_attention": {"achieved": round(attn_gbs, 1), "unit": "GB/s",
                             "frac": round(attn_gbs / HBM_PEAK_GBS, 4),
                             "bytes_per_launch": attn_bytes, "us_per_launch": round(attn_us, 2)},
    }

    if not args.no_cpu_baseline:
        cpu_us, cores, ref_sels, ref_out = cpu_baseline(wl, args.cpu_reps)
        result["cpu_baseline"] = {
            "value": round(cpu_us, 1), "unit": "us", "cores": cores, "kind": "port",
            "sample": f"the full {wl.name} layer, median of {args.cpu_reps} repetitions "
                      "after one warm-up (PyTorch CPU oracle)"}
        # Parity of this very run against the oracle.
        S = [int(x) for x in layer.sel_len.tolist()]
        same = all(torch.equal(layer.sel[b, :S[b]].cpu(), ref_sels[b]) for b in range(B))
        err = (layer.out.cpu().float() - ref_out.float()).abs().max().item()
        result["parity"] = {"selected_slots_identical": bool(same),
                            "attn_max_abs_err": round(err, 5)}
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
