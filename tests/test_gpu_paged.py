"""Paged KV store / table append (pages of 16 tokens, fresh pages from a device-side
free list) against ``oracle.store``, then the paths that grow a paged cache: a decode
trace and a chunked prefill, step by step against the oracle on the same pools."""

import pytest
import torch

import oracle
from tokenselect_amd import ops, workloads
from helpers import assert_attention_close, assert_index_sets_match, say

pytestmark = pytest.mark.gpu

LLAMA = dict(num_heads=32, num_kv_heads=8, rope_theta=5e5)
SMALL = dict(num_heads=8, num_kv_heads=2, rope_theta=1e4)


def _pool_state(pool: ops.PagePool):
    return pool.free_pages[:int(pool.free_count)].cpu().tolist()


def _mirror(wl, extra_tokens):
    """CPU twins of a workload's tables, with room for `extra_tokens` more per request."""
    ps = wl.cfg.page_size
    pages = -(-(max(wl.seq_lens) + extra_tokens) // ps)
    table = torch.full((len(wl.seq_lens), pages), -1, dtype=torch.int32)
    table[:, :wl.table.shape[1]] = wl.table.cpu()
    return table


def test_kv_store_paged(dev):
    """Lengths on and off page boundaries, a full table, fourteen steps in a row: table,
    lengths, free list and the rows in the pools against the oracle."""
    say("paged kv_store: page 16, B=6")
    ps, lens = 16, [32, 15, 16, 31, 100, 47]
    wl = workloads.build("paged", SMALL, lens, [8] * 6, ps, dev, seed=3, n_init=2, n_local=4,
                         extra_pages=4)    # five pages are wanted: the last request finds none
    c = wl.cfg
    max_tokens = 112                         # request 4 (100 tokens) fills up during the test
    table = torch.full((6, max_tokens // ps), -1, dtype=torch.int32, device=dev)
    table[:, :wl.table.shape[1]] = wl.table
    ref_table, ref_lens = table.cpu().clone(), list(lens)
    seq = wl.seq_lens_dev.clone()
    pool = ops.PagePool.of(wl.free_pages)
    ref_free = wl.free_pages.cpu().tolist()
    kc, vc = wl.k_pool.cpu().clone(), wl.v_pool.cpu().clone()
    g = torch.Generator(device=dev).manual_seed(4)
    for step in range(14):
        k = torch.randn((6, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
        v = torch.randn((6, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
        ops.kv_store(c, k, v, None, wl.k_pool, wl.v_pool, table, seq, pages=pool)
        torch.cuda.synchronize()
        slots = oracle.store.append_token_paged(ref_table, ref_lens, ref_free, ps, max_tokens,
                                                wl.k_pool.shape[0])
        for b, s in enumerate(slots):
            if s is not None:
                kc[s], vc[s] = k[b].cpu(), v[b].cpu()
        assert seq.cpu().tolist() == ref_lens, f"step {step}"
        assert torch.equal(table.cpu(), ref_table), f"step {step}"
        assert _pool_state(pool) == ref_free and int(pool.ticket) == 0, f"step {step}"
    assert torch.equal(wl.k_pool.cpu(), kc) and torch.equal(wl.v_pool.cpu(), vc)
    assert ref_lens[4] == max_tokens          # the full table stopped growing
    assert None in slots                      # and the list ran dry for somebody
    assert ref_free == []


def test_kv_store_paged_across_wavefront_rounds(dev):
    """A batch of 150: the plan walks the requests 64 at a time and carries the rank of the
    requests that need a page from one round to the next.  Requests on page boundaries sit in
    all three rounds, the list runs dry inside the third, and one entry of the list is a page
    beyond the pool (dropped with its request left untouched, the stack staying contiguous).
    Table, lengths, free list and pool rows against the oracle, three steps in a row."""
    B, ps, pages_per_req = 150, 16, 6
    say(f"paged kv_store: B={B} across rounds of 64")
    c = ops.LayerConfig(num_heads=8, num_kv_heads=2, page_size=ps, n_init=2, n_local=4, top_k=8,
                        rope_theta=1e4)
    g = torch.Generator().manual_seed(11)
    lens = torch.randint(1, 70, (B,), generator=g)
    lens[torch.randperm(B, generator=g)[:60]] //= ps
    lens = (lens.clamp_min(0) * 1).tolist()
    lens = [L * ps if i % 5 == 0 else L for i, L in enumerate(lens)]     # many on a boundary
    lens = [min(L, pages_per_req * ps - 2) for L in lens]
    total_pages = B * pages_per_req + 40
    perm = torch.randperm(total_pages, generator=g).int()
    table = torch.full((B, pages_per_req), -1, dtype=torch.int32)
    at = 0
    for b, L in enumerate(lens):
        used = -(-L // ps)
        table[b, :used] = perm[at:at + used]
        at += used
    need_now = sum(1 for L in lens if L % ps == 0)
    free = perm[at:at + need_now - 7].clone()            # seven requests too few
    free[len(free) // 2] = total_pages + 5               # a page beyond the pool
    pool_rows = total_pages * ps
    k_pool = torch.zeros((pool_rows, 2, 128), dtype=torch.bfloat16, device=dev)
    v_pool = torch.zeros_like(k_pool)
    table_d, seq = table.to(dev), torch.tensor(lens, dtype=torch.int32, device=dev)
    pool = ops.PagePool.of(free.to(dev))
    ref_table, ref_lens, ref_free = table.clone(), list(lens), free.tolist()
    kc, vc = k_pool.cpu().clone(), v_pool.cpu().clone()
    gd = torch.Generator(device=dev).manual_seed(12)
    refused = 0
    for step in range(3):
        k = torch.randn((B, 2, 128), generator=gd, device=dev).bfloat16()
        v = torch.randn((B, 2, 128), generator=gd, device=dev).bfloat16()
        ops.kv_store(c, k, v, None, k_pool, v_pool, table_d, seq, pages=pool)
        torch.cuda.synchronize()
        slots = oracle.store.append_token_paged(ref_table, ref_lens, ref_free, ps, pages_per_req * ps,
                                                pool_rows)
        for b, s_ in enumerate(slots):
            if s_ is not None:
                kc[s_], vc[s_] = k[b].cpu(), v[b].cpu()
        refused += sum(1 for s_ in slots if s_ is None)
        assert seq.cpu().tolist() == ref_lens, f"step {step}"
        assert torch.equal(table_d.cpu(), ref_table), f"step {step}"
        assert _pool_state(pool) == ref_free and int(pool.ticket) == 0, f"step {step}"
    assert refused >= 8 and ref_free == []
    assert torch.equal(k_pool.cpu(), kc) and torch.equal(v_pool.cpu(), vc)


def test_qkv_store_paged_equals_the_unfused_store(dev):
    say("paged qkv_store against F.linear + paged kv_store")
    ps, lens = 16, [16, 5, 48, 33]
    wl = workloads.build("paged", SMALL, lens, [8] * 4, ps, dev, seed=6, n_init=2, n_local=4,
                         extra_pages=4)
    c = wl.cfg
    hidden = 256
    g = torch.Generator(device=dev).manual_seed(7)
    x = torch.randn((4, hidden), generator=g, device=dev).bfloat16()
    n_out = (c.num_heads + 2 * c.num_kv_heads) * 128
    w = (torch.randn((n_out, hidden), generator=g, device=dev) * hidden ** -0.5).bfloat16()
    pages = -(-(max(lens) + 1) // ps)
    t1 = torch.full((4, pages), -1, dtype=torch.int32, device=dev)
    t1[:, :wl.table.shape[1]] = wl.table
    t2 = t1.clone()
    s1, s2 = wl.seq_lens_dev.clone(), wl.seq_lens_dev.clone()
    k1, v1, k2, v2 = wl.k_pool.clone(), wl.v_pool.clone(), wl.k_pool.clone(), wl.v_pool.clone()
    p1, p2 = ops.PagePool.of(wl.free_pages), ops.PagePool.of(wl.free_pages)
    q = ops.qkv_store(c, x, w, None, None, k1, v1, t1, s1, pages=p1)
    y = torch.nn.functional.linear(x.double(), w.double())
    hd, kvd = c.num_heads * 128, c.num_kv_heads * 128
    ops.kv_store(c, y[:, hd:hd + kvd].bfloat16().contiguous(), y[:, hd + kvd:].bfloat16().contiguous(),
                 None, k2, v2, t2, s2, pages=p2)
    torch.cuda.synchronize()
    assert torch.equal(t1, t2) and torch.equal(s1, s2) and _pool_state(p1) == _pool_state(p2)
    assert int(p1.ticket) == 0 and s1.tolist() == [L + 1 for L in lens]
    assert (q.double() - y[:, :hd]).abs().max().item() <= 2 ** -7 * y[:, :hd].abs().max().item()
    # rows land in the same slots, within one bf16 rounding of each other
    changed = (k1 != wl.k_pool).flatten(1).any(1) | (k2 != wl.k_pool).flatten(1).any(1)
    assert int(changed.sum()) == 4
    assert (k1.float() - k2.float()).abs().max().item() <= 2 ** -6 * k2.float().abs().max().item()
    assert (v1.float() - v2.float()).abs().max().item() <= 2 ** -6 * v2.float().abs().max().item()


def test_kv_store_chunk_paged(dev):
    say("paged kv_store_chunk: chunks of 80, 45, 3, 40 rows on pages of 16")
    ps, L0 = 16, 37
    wl = workloads.build("paged", SMALL, [L0], [8], ps, dev, seed=8, n_init=2, n_local=4,
                         extra_pages=9)
    c = wl.cfg
    max_tokens = 192
    table = torch.full((1, max_tokens // ps), -1, dtype=torch.int32, device=dev)
    table[:, :wl.table.shape[1]] = wl.table
    ref_row, L = table[0].cpu().clone(), L0
    seq = wl.seq_lens_dev.clone()
    pool = ops.PagePool.of(wl.free_pages)
    ref_free = wl.free_pages.cpu().tolist()
    kc, vc = wl.k_pool.cpu().clone(), wl.v_pool.cpu().clone()
    g = torch.Generator(device=dev).manual_seed(9)
    for rows in (80, 45, 3, 40):              # the last one runs out of pages and of table
        k = torch.randn((rows, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
        v = torch.randn((rows, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
        ops.kv_store_chunk(c, k, v, None, wl.k_pool, wl.v_pool, table[0], seq, pages=pool)
        torch.cuda.synchronize()
        slots, L = oracle.store.append_chunk_paged(ref_row, L, rows, ref_free, ps, max_tokens)
        for r, s in enumerate(slots):
            kc[s], vc[s] = k[r].cpu(), v[r].cpu()
        assert int(seq) == L and torch.equal(table[0].cpu(), ref_row), rows
        assert _pool_state(pool) == ref_free and int(pool.ticket) == 0, rows
    assert L < L0 + 80 + 45 + 3 + 40          # something was dropped
    assert torch.equal(wl.k_pool.cpu(), kc) and torch.equal(wl.v_pool.cpu(), vc)


@pytest.mark.parametrize("fused", [True, False], ids=["fused", "separate"])
def test_decode_trace_on_a_paged_cache(dev, fused):
    """40 decode steps of a Llama-3-8B-shaped layer on pages of 16 tokens: every step
    appends through the page pool and then selects and attends; tables, selection and
    attention output against the oracle on CPU twins of the pools."""
    say(f"paged decode trace, 40 steps, fused={fused}")
    previous = ops.set_fused_select(fused)
    try:
        ps, lens, steps = 16, [1500, 617, 90], 40
        wl = workloads.build("paged", LLAMA, lens, [128] * 3, ps, dev, seed=10, n_init=16, n_local=64,
                             top_k=128, extra_pages=3 * 4)
        c, B = wl.cfg, 3
        ref_table = _mirror(wl, steps)
        table = ref_table.to(dev)
        ref_lens, seq = list(lens), wl.seq_lens_dev.clone()
        pool = ops.PagePool.of(wl.free_pages)
        ref_free = wl.free_pages.cpu().tolist()
        kc, vc = wl.k_pool.cpu().clone(), wl.v_pool.cpu().clone()
        layer = ops.DecodeLayer(c, B, max(lens) + steps, dev)
        g = torch.Generator(device=dev).manual_seed(11)
        for t in range(steps):
            q = torch.randn((B, c.num_heads * 128), generator=g, device=dev).bfloat16()
            k = torch.randn((B, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
            v = torch.randn((B, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
            ops.kv_store(c, k, v, None, wl.k_pool, wl.v_pool, table, seq, pages=pool)
            out, sel, sel_pos, sel_len = layer(q, wl.k_pool, wl.v_pool,
                                               ops.Batch(seq, table, max(lens) + t + 1))
            torch.cuda.synchronize()
            for b, s in enumerate(oracle.store.append_token_paged(ref_table, ref_lens, ref_free, ps,
                                                                  table.shape[1] * ps,
                                                                  wl.k_pool.shape[0])):
                kc[s], vc[s] = k[b].cpu(), v[b].cpu()
            assert torch.equal(table.cpu(), ref_table) and seq.cpu().tolist() == ref_lens
            tabs = [oracle.select.expand_page_table(ref_table[b], ref_lens[b], ps) for b in range(B)]
            details = []
            ref_sel, ref_out = oracle.layer.decode_layer(
                q.cpu(), kc, vc, tabs, ref_lens, c.num_heads, 128, c.n_init, c.n_local, [128] * B,
                c.rope_theta, c.rope_scale, 128 ** -0.5, details=details)
            step_wl = workloads.Workload("step", c, q, wl.k_pool, wl.v_pool, table, ref_lens, seq,
                                         [128] * B)
            for b in range(B):
                S = int(sel_len[b])
                assert S == ref_sel[b].shape[0]
                if details[b]:
                    assert_index_sets_match(sel_pos[b, c.n_init:S - c.n_local].cpu(),
                                            details[b]["top_pos"], details[b]["votes"], c.n_init,
                                            f"step {t} b={b}")
                else:
                    assert torch.equal(sel[b, :S].cpu(), ref_sel[b])
                assert_attention_close(step_wl, b, out[b], sel[b, :S], ref_sel[b], ref_out[b],
                                       f"step {t} b={b}")
        assert len(ref_free) == 12 - 3 * 3 and _pool_state(pool) == ref_free
    finally:
        ops.set_fused_select(previous)


def test_prefill_chunks_on_a_paged_cache(dev):
    """Three prefill chunks (the last one ragged) on pages of 16 tokens: paged chunk store,
    then the chunk's selection and causal attention against the oracle."""
    say("paged prefill, 3 chunks of <= 64 rows")
    ps, L0, chunk, T, top_k = 16, 700, 64, 150, 96
    wl = workloads.build("paged", LLAMA, [L0], [top_k], ps, dev, seed=12, n_init=8, n_local=chunk,
                         top_k=top_k, extra_pages=11)
    c = wl.cfg
    g = torch.Generator(device=dev).manual_seed(13)
    q = torch.randn((T, c.num_heads * 128), generator=g, device=dev).bfloat16()
    k_new = torch.randn((T, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
    v_new = torch.randn((T, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
    ref_row = _mirror(wl, T)[0]
    table = ref_row.view(1, -1).to(dev)
    seq = wl.seq_lens_dev.clone()
    pool = ops.PagePool.of(wl.free_pages)
    ref_free = wl.free_pages.cpu().tolist()
    kc, vc = wl.k_pool.cpu().clone(), wl.v_pool.cpu().clone()
    layer = ops.PrefillChunk(c, L0 + T, dev, max_rows=chunk)
    L = L0
    for start in range(0, T, chunk):
        end = min(start + chunk, T)
        m = end - start
        ops.kv_store_chunk(c, k_new[start:end], v_new[start:end], None, wl.k_pool, wl.v_pool, table[0],
                           seq, pages=pool)
        slots, L = oracle.store.append_chunk_paged(ref_row, L, m, ref_free, ps, table.shape[1] * ps)
        out, sel, sel_pos, sel_len = layer(q[start:end].contiguous(), wl.k_pool, wl.v_pool,
                                           ops.Batch(seq, table, L))
        torch.cuda.synchronize()
        assert int(seq) == L and torch.equal(table[0].cpu(), ref_row)
        for r, s in enumerate(slots):
            kc[s], vc[s] = k_new[start + r].cpu(), v_new[start + r].cpu()
        tab = oracle.select.expand_page_table(ref_row, L, ps)
        qf = ops.fingerprint(c, q[start:end].view(m, c.num_heads, 128).contiguous(), layer.cos,
                             layer.sin).cpu()
        d = {}
        ref_slots, ref_out = oracle.prefill.prefill_chunk(
            q[start:end].cpu(), kc, vc, tab, L, c.num_heads, 128, c.n_init, c.n_local, top_k,
            c.rope_theta, c.rope_scale, 128 ** -0.5, detail=d, qf_override=qf)
        S = int(sel_len[0])
        assert S == ref_slots.shape[0]
        pos = sel_pos[0, :S].cpu()
        assert_index_sets_match(pos[c.n_init:c.n_init + top_k], d["top_pos"], d["votes"], c.n_init,
                                f"chunk at {start}")
        assert torch.equal(sel[0, :S].cpu(), tab[pos.long()])
        if not torch.equal(sel[0, :S].cpu(), ref_slots):
            ref_out = oracle.prefill.sparse_prefill_attention(
                q[start:end].cpu().view(m, c.num_heads, 128), kc, vc, sel[0, :S].cpu(), 128 ** -0.5,
                c.rope_theta, c.rope_scale).reshape(m, -1)
        assert (out.cpu().float() - ref_out.float()).abs().max().item() <= 2e-2, start
