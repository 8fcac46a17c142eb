"""GPU parity of the patch-layer mirror (the drop-in boundary) and of the
selection cache against the oracle, on multi-step decode traces."""

import pytest
import torch

import oracle
from tokenselect_amd import ops, workloads
from tokenselect_amd.patcher import sglang_standins as sg
from tokenselect_amd.patcher import token_retrieval as tr
from helpers import assert_index_sets_match, say

pytestmark = pytest.mark.gpu


def test_patched_decode_forward_trace(dev):
    """Prefill by direct stores, then decode steps through the patched
    RadixAttention.forward: store -> select -> attend, crossing from the dense
    fallback (short context) into selection."""
    say("patched decode forward trace: 2 layers, H8/kv2, top_k 32")
    H, Hkv, D, layers, hidden = 8, 2, 128, 2, 256
    n_init, n_local, top_k = 4, 8, 32
    tr.patch(rope_base=1e4, rope_scale=1, rope_model="ROPE_LLAMA", max_n_tokens=512, top_k=top_k,
             n_init=n_init, n_local=n_local)
    g = torch.Generator(device=dev).manual_seed(5)
    pool = sg.TokenToKVPool(1024, torch.bfloat16, Hkv, D, layers, dev)
    runner = sg.ModelRunner(model_config=sg.ModelConfig(layers, D, H, Hkv), token_to_kv_pool=pool,
                            dtype=torch.bfloat16)
    assert isinstance(runner, sg.ModelRunner) and hasattr(runner, "req_to_token_retriever")
    retriever = runner.req_to_token_retriever.get_token_retriever("req-0")
    slots = torch.randperm(1024, generator=g, device=dev).to(torch.int32)
    mods = [sg.Attention(hidden, H, Hkv, D, l, device=dev) for l in range(layers)]

    prefill = 30
    for l in range(layers):
        pool.k_buffer[l][slots[:prefill].long()] = torch.randn(prefill, Hkv, D, generator=g,
                                                               device=dev).bfloat16()
        pool.v_buffer[l][slots[:prefill].long()] = torch.randn(prefill, Hkv, D, generator=g,
                                                               device=dev).bfloat16()
        retriever.add_k_cache(slots[:prefill], l)

    saw_dense = saw_sparse = False
    for step in range(40):
        L = prefill + step + 1
        loc = slots[L - 1:L].contiguous()
        meta = sg.InputMetadata(sg.ForwardMode.DECODE, retriever, pool, loc)
        x = torch.randn(1, hidden, generator=g, device=dev).bfloat16()
        for l, mod in enumerate(mods):
            qkv, _ = mod.qkv_proj(x)
            q, k, v = qkv.split([mod.q_size, mod.kv_size, mod.kv_size], dim=-1)
            got = mod.attn(q.contiguous(), k.contiguous(), v.contiguous(), meta)
            assert got.shape == (1, H * D)
            assert retriever.num_tokens[l] == L
            kc, vc = pool.k_buffer[l].cpu(), pool.v_buffer[l].cpu()
            tab = retriever.get_all_tokens(l).cpu()
            assert tab[-1].item() == loc.item()
            assert torch.equal(kc[loc.item()].reshape(-1), k.cpu().reshape(-1))
            d = []
            ref_sel, ref_out = oracle.layer.decode_layer(q.cpu(), kc, vc, [tab], [L], H, D, n_init,
                                                         n_local, [top_k], 1e4, 1, D ** -0.5,
                                                         details=d)
            dense = oracle.select.is_dense(L, n_init, n_local, top_k)
            saw_dense |= dense
            saw_sparse |= not dense
            err = (got.cpu().float() - ref_out.float()).abs().max().item()
            assert err <= 2e-2, f"step {step} layer {l} (L={L}, dense={dense}): {err}"
            if not dense:
                sel = retriever.retrieval_indices(q.contiguous(), l, n_init, n_local, top_k)
                assert sel.dtype == torch.int32 and sel.shape[0] == n_init + top_k + n_local
                assert torch.equal(sel.cpu(), ref_sel[0]), f"step {step} layer {l}: slots differ"
            else:
                assert retriever.retrieval_indices(q.contiguous(), l, n_init, n_local, top_k) is None
    assert saw_dense and saw_sparse

    # the module-level forward: QKV projection -> attention (no rotary) -> output projection
    L = prefill + 41
    loc = slots[L - 1:L].contiguous()
    meta = sg.InputMetadata(sg.ForwardMode.DECODE, retriever, pool, loc)
    x = torch.randn(1, hidden, generator=g, device=dev).bfloat16()
    y = mods[0](None, x, meta)
    assert y.shape == (1, hidden) and retriever.num_tokens[0] == L
    qkv, _ = mods[0].qkv_proj(x)
    q = qkv[:, :mods[0].q_size]
    _, ref_out = oracle.layer.decode_layer(q.cpu(), pool.k_buffer[0].cpu(), pool.v_buffer[0].cpu(),
                                           [retriever.get_all_tokens(0).cpu()], [L], H, D, n_init,
                                           n_local, [top_k], 1e4, 1, D ** -0.5)
    ref_y = mods[0].o_proj(ref_out.to(dev))[0]
    assert (y.float() - ref_y.float()).abs().max().item() <= 3e-2


def test_get_topk_tokens_and_paged_matmul_mirror(dev):
    say("mirror get_topk_tokens / paged_matmul")
    tr.patch(rope_base=1e4, top_k=16, n_init=2, n_local=4, max_n_tokens=2048)
    H, Hkv, D = 8, 2, 128
    g = torch.Generator().manual_seed(9)
    kbuf = torch.randn(600, Hkv, D, generator=g).bfloat16()
    pool = sg.TokenToKVPool(599, torch.bfloat16, Hkv, D, 1, dev)
    pool.k_buffer[0].copy_(kbuf)
    r = tr.TokenRetriever(1, D, H, Hkv, Hkv * D, 2048, torch.bfloat16, dev, token_to_kv_pool=pool,
                          rotary_embedding=tr.RotaryEmbedding(D, 1e4, 1, dev))
    qf = torch.randn(H * D, generator=g).bfloat16()
    idx = torch.randperm(600, generator=g)[:500].int()
    got = r.get_topk_tokens(qf.to(dev), pool.get_key_buffer(0), 16, idx.to(dev))
    assert got.dtype == torch.int64 and got.shape == (16,)
    ref, s, c = oracle.select.get_topk_tokens(qf, kbuf, 16, idx, D, return_all=True)
    assert_index_sets_match(got.cpu() + 0, ref, c, 0, "get_topk_tokens")
    scores = torch.empty((H, 500), dtype=torch.bfloat16, device=dev)
    tr.paged_matmul(qf.view(H, D).to(dev), pool.get_key_buffer(0), idx.to(dev), scores, 500, H, Hkv, D)
    assert ((scores.float().cpu() - s).abs() <= s.abs() * 2.0 ** -8 + 1e-6).all()
    rot = tr.RotaryEmbedding(D, 1e4, 1.0, dev)
    x = torch.randn(3, H, D, generator=g).bfloat16()
    pos = torch.tensor([4, 5, 6])
    assert torch.equal(rot(x.to(dev), pos.to(dev)).cpu(), oracle.rope.apply(x, pos, 1e4, 1.0))


@pytest.mark.parametrize("anchor_jump", [0.1])
def test_selection_cache_trace(dev, anchor_jump):
    """Batched decode trace with the selection cache: hit flags, reused middle
    segments, sliding local windows and counters against the oracle's state
    machine (AR(1) queries, rho 0.95, occasional jumps)."""
    B, L0, steps, top_k = 3, 1500, 24, 64
    say(f"selection-cache trace B={B} L0={L0} steps={steps}")
    wl = workloads.build("trace", workloads.LLAMA3_8B, [L0] * B, [top_k] * B, 1, dev, seed=13,
                         n_init=8, n_local=32, top_k=top_k, extra_pages=B * steps)
    c = wl.cfg
    qs = workloads.ar1_queries(B, c.num_heads * c.head_dim, steps, dev, seed=13, rho=0.95,
                               jump_p=anchor_jump)
    table = torch.zeros((B, L0 + steps), dtype=torch.int32, device=dev)
    table[:, :L0] = wl.table
    seq = wl.seq_lens_dev.clone()
    free = torch.arange(B * L0, B * (L0 + steps), dtype=torch.int32, device=dev).view(steps, B)
    cache = ops.SelectionCache.allocate(c, B, dev)
    layer = ops.DecodeLayer(c, B, L0 + steps, dev)
    g = torch.Generator(device=dev).manual_seed(99)

    ref_caches = [oracle.selcache.SelectionCache() for _ in range(B)]
    kc, vc = wl.k_pool.cpu(), wl.v_pool.cpu()
    total_hits = 0
    for t in range(steps):
        k_new = torch.randn(B, c.num_kv_heads * 128, generator=g, device=dev).bfloat16()
        v_new = torch.randn(B, c.num_kv_heads * 128, generator=g, device=dev).bfloat16()
        ops.kv_store(c, k_new, v_new, free[t].contiguous(), wl.k_pool, wl.v_pool, table, seq)
        L = L0 + t + 1
        bt = ops.Batch(seq, table, L)
        out, sel, sel_pos, sel_len = layer(qs[t].contiguous(), wl.k_pool, wl.v_pool, bt, cache)
        torch.cuda.synchronize()
        kc[free[t].cpu().long()] = k_new.cpu().view(B, c.num_kv_heads, 128)
        vc[free[t].cpu().long()] = v_new.cpu().view(B, c.num_kv_heads, 128)
        tab_cpu = table.cpu()
        for b in range(B):
            S = int(sel_len[b])
            assert S == c.max_sel
            tab = tab_cpu[b, :L]
            q = qs[t, b].cpu().view(1, -1)
            qf = oracle.rope.scoring_query(q, c.num_heads, 128, c.n_local, c.rope_theta, 1.0)
            d = {}

            def run_select():
                oracle.select.retrieval_indices(q, kc, tab, L, c.num_heads, 128, c.n_init, c.n_local,
                                                top_k, c.rope_theta, 1.0, detail=d)
                return d["top_pos"]

            ref_top, ref_hit = ref_caches[b].step(qf, run_select)
            total_hits += int(ref_hit)
            pos = sel_pos[b, :S].cpu()
            mid = pos[c.n_init:c.n_init + top_k]
            if ref_hit:
                assert torch.equal(mid.long(), ref_top), f"step {t} req {b}: hit must reuse the cache"
            else:
                assert_index_sets_match(mid, ref_top, d["votes"], c.n_init, f"step {t} req {b}")
                ref_caches[b].top_cached = mid.long().clone()   # follow the GPU's tie choice
            assert pos[-c.n_local:].tolist() == list(range(L - c.n_local, L))   # window slides
            assert torch.equal(sel[b, :S].cpu(), tab[pos.long()])
            ref_out = oracle.attend.sparse_decode_attention(
                qs[t, b].cpu().view(c.num_heads, 128), kc, vc, tab[pos.long()], 128 ** -0.5,
                c.rope_theta)
            assert (out[b].cpu().float() - ref_out.reshape(-1).float()).abs().max().item() <= 2e-2
    counters = cache.counters.cpu()
    assert counters[:, 1].tolist() == [steps] * B
    assert int(counters[:, 0].sum()) == total_hits
    assert 0 < total_hits < B * steps, "the trace must exercise both hits and misses"


@pytest.mark.parametrize("defaults", [False, True], ids=["chunk 32 in a window of 32", "patch() defaults"])
def test_patched_extend_forward(dev, defaults):
    """Chunked prefill through the patched RadixAttention.forward in EXTEND mode: a
    prompt of three chunks (the last one ragged) on an empty cache, then one more
    extend on top; every chunk against the oracle's extend loop on the same pools.
    Second case: the reference's own patch() defaults (top_k 16, n_init 1, n_local 16,
    tr.py:885-894) with its 512-row chunks, which are far longer than the local window."""
    H, Hkv, D, layers = 8, 2, 128, 2
    if defaults:
        n_init, n_local, top_k, chunk, rope_base, prompts = 1, 16, 16, 512, 1e6, (600, 45)
        say("patched extend forward: 2 layers, H8/kv2, patch() defaults, chunk 512")
        tr.patch()
    else:
        n_init, n_local, top_k, chunk, rope_base, prompts = 4, 32, 24, 32, 1e4, (80, 45)
        say("patched extend forward: 2 layers, H8/kv2, chunk 32, top_k 24")
        tr.patch(rope_base=1e4, rope_scale=1, rope_model="ROPE_LLAMA", max_n_tokens=512, top_k=top_k,
                 n_init=n_init, n_local=n_local)
    tr.PREFILL_CHUNK_SIZE = chunk
    try:
        g = torch.Generator(device=dev).manual_seed(17)
        pool = sg.TokenToKVPool(1024, torch.bfloat16, Hkv, D, layers, dev)
        runner = sg.ModelRunner(model_config=sg.ModelConfig(layers, D, H, Hkv),
                                token_to_kv_pool=pool, dtype=torch.bfloat16)
        retriever = runner.req_to_token_retriever.get_token_retriever("req-extend")
        slots = torch.randperm(1024, generator=g, device=dev).to(torch.int32)
        attns = [sg.RadixAttention(H, D, D ** -0.5, Hkv, layer_id=l) for l in range(layers)]
        ref_k = [pool.k_buffer[l].cpu().clone() for l in range(layers)]
        ref_v = [pool.v_buffer[l].cpu().clone() for l in range(layers)]
        ref_tab = [torch.zeros(1024, dtype=torch.int32) for _ in range(layers)]
        L = 0
        for T in prompts:
            loc = slots[L:L + T].contiguous()
            meta = sg.InputMetadata(sg.ForwardMode.EXTEND, retriever, pool, loc)
            for l, attn in enumerate(attns):
                q = torch.randn(T, H * D, generator=g, device=dev).bfloat16()
                k = torch.randn(T, Hkv * D, generator=g, device=dev).bfloat16()
                v = torch.randn(T, Hkv * D, generator=g, device=dev).bfloat16()
                got = attn.forward(q, k, v, meta)
                torch.cuda.synchronize()
                assert got.shape == (T, H * D) and retriever.num_tokens[l] == L + T
                assert torch.equal(retriever.get_all_tokens(l).cpu(), slots[:L + T].cpu())
                # the oracle follows the device's chunk fingerprints (its own fp32 mean may
                # round a bf16 element the other way), so that every row is compared
                pf = retriever._layers[("prefill", attn.scaling, attn.logit_cap)]
                qfs = [ops.fingerprint(pf.cfg, q[s:min(s + chunk, T)].view(-1, H, D).contiguous(),
                                       pf.cos, pf.sin).cpu() for s in range(0, T, chunk)]
                details = []
                ref = oracle.prefill.prefill(q.cpu(), k.cpu().view(T, Hkv, D), v.cpu().view(T, Hkv, D),
                                             ref_k[l], ref_v[l], ref_tab[l], L, loc.cpu(), H, D, n_init,
                                             n_local, top_k, rope_base, 1, D ** -0.5, chunk=chunk,
                                             details=details, qf_overrides=qfs)
                assert torch.equal(pool.k_buffer[l].cpu(), ref_k[l])
                err = (got.cpu().float() - ref.float()).abs().max().item()
                assert err <= 2e-2, f"extend T={T} layer {l}: max abs err {err:.4f}"
            L += T
    finally:
        tr.PREFILL_CHUNK_SIZE = 512


def test_patched_decode_forward_for_a_batch(dev):
    """Two requests prefilled one by one through the patched extend forward, then decoded
    together through the patched decode forward with a BatchTokenRetriever: per request
    the store, the table and the attention output against the oracle."""
    say("patched decode forward, batch of 2")
    H, Hkv, D, layers = 8, 2, 128, 2
    n_init, n_local, top_k, chunk = 4, 32, 24, 32
    tr.patch(rope_base=1e4, rope_scale=1, rope_model="ROPE_LLAMA", max_n_tokens=512, top_k=top_k,
             n_init=n_init, n_local=n_local)
    tr.PREFILL_CHUNK_SIZE = chunk
    try:
        g = torch.Generator(device=dev).manual_seed(23)
        pool = sg.TokenToKVPool(1024, torch.bfloat16, Hkv, D, layers, dev)
        runner = sg.ModelRunner(model_config=sg.ModelConfig(layers, D, H, Hkv),
                                token_to_kv_pool=pool, dtype=torch.bfloat16)
        owner = runner.req_to_token_retriever
        slots = torch.randperm(1024, generator=g, device=dev).to(torch.int32)
        attns = [sg.RadixAttention(H, D, D ** -0.5, Hkv, layer_id=l) for l in range(layers)]
        prompts, used, singles = [150, 70], 0, []
        for T in prompts:                      # prefill, one request at a time
            r = owner.new_token_retriever()
            loc = slots[used:used + T].contiguous()
            meta = sg.InputMetadata(sg.ForwardMode.EXTEND, r, pool, loc)
            for attn in attns:
                q = torch.randn(T, H * D, generator=g, device=dev).bfloat16()
                k = torch.randn(T, Hkv * D, generator=g, device=dev).bfloat16()
                v = torch.randn(T, Hkv * D, generator=g, device=dev).bfloat16()
                attn.forward(q, k, v, meta)
            used += T
            singles.append(r)
        batch = owner.get_batch_token_retriever(("a", "b"), singles)
        assert batch is owner.get_batch_token_retriever(("a", "b"))       # same batch, same object
        with pytest.raises(ValueError):
            owner.get_batch_token_retriever(("a", "c"))                    # new composition, no tables
        lens = list(prompts)
        for step in range(6):
            loc = slots[used:used + 2].contiguous()
            used += 2
            meta = sg.InputMetadata(sg.ForwardMode.DECODE, batch, pool, loc, batch_size=2)
            for l, attn in enumerate(attns):
                q = torch.randn(2, H * D, generator=g, device=dev).bfloat16()
                k = torch.randn(2, Hkv * D, generator=g, device=dev).bfloat16()
                v = torch.randn(2, Hkv * D, generator=g, device=dev).bfloat16()
                got = attn.forward(q, k, v, meta)
                torch.cuda.synchronize()
                assert got.shape == (2, H * D)
                kc, vc = pool.k_buffer[l].cpu(), pool.v_buffer[l].cpu()
                tabs = [t.cpu() for t in batch.get_all_tokens(l)]
                assert [t.shape[0] for t in tabs] == [n + 1 for n in lens]
                for b in range(2):
                    assert tabs[b][-1].item() == loc[b].item()
                    assert torch.equal(kc[loc[b].item()].reshape(-1), k[b].cpu())
                _, ref_out = oracle.layer.decode_layer(q.cpu(), kc, vc, tabs, [n + 1 for n in lens], H, D,
                                                       n_init, n_local, [top_k] * 2, 1e4, 1, D ** -0.5)
                err = (got.cpu().float() - ref_out.float()).abs().max().item()
                assert err <= 2e-2, f"step {step} layer {l}: {err}"
            lens = [n + 1 for n in lens]
        with pytest.raises(NotImplementedError):                           # wrong number of rows
            attns[0].forward(torch.zeros(3, H * D, dtype=torch.bfloat16, device=dev), None, None, meta)
    finally:
        tr.PREFILL_CHUNK_SIZE = 512
