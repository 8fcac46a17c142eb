"""GPU parity of the chunked-prefill path against the CPU oracle, through the C ABI:
chunk fingerprint within one bf16 ulp (fp32 summation order), selection identical
for the same fingerprint up to ties at the k-th vote, causal sparse attention
within 2e-2 absolute in bf16."""

import pytest
import torch

import oracle
from tokenselect_amd import ops, workloads
from helpers import assert_index_sets_match, cpu_tabs, say

pytestmark = pytest.mark.gpu

SHAPES = [
    dict(num_heads=32, num_kv_heads=8, rope_theta=5e5),   # Llama-3-8B
    dict(num_heads=28, num_kv_heads=4, rope_theta=1e6),   # Qwen2-7B
    dict(num_heads=8, num_kv_heads=1, rope_theta=1e4),
    dict(num_heads=4, num_kv_heads=2, rope_theta=1e4),
    dict(num_heads=8, num_kv_heads=8, rope_theta=1e4),
    dict(num_heads=24, num_kv_heads=8, rope_theta=5e5),   # Llama-3.2-3B: three query heads per KV head
    dict(num_heads=12, num_kv_heads=2, rope_theta=1e6),   # Qwen2-1.5B: six
    dict(num_heads=20, num_kv_heads=4, rope_theta=1e4),   # five
]
IDS = [f"H{s['num_heads']}kv{s['num_kv_heads']}" for s in SHAPES]


def _sm(c):
    return c.sm_scale if c.sm_scale is not None else c.head_dim ** -0.5


@pytest.mark.parametrize("rows", [1, 37, 512])
def test_fingerprint(dev, rows):
    say(f"chunk fingerprint rows={rows}")
    g = torch.Generator().manual_seed(rows)
    H, n_local = 6, 40
    cfg = ops.LayerConfig(num_heads=8, num_kv_heads=8, n_local=n_local, rope_theta=5e5)
    q = torch.randn(rows, 8, 128, generator=g).bfloat16()
    cos, sin = ops.rope_tables(128, 5e5, 1.0, n_local + rows, dev)
    got = ops.fingerprint(cfg, q.to(dev), cos, sin).cpu().float().reshape(-1)
    ref = oracle.rope.scoring_query(q.view(rows, -1), 8, 128, n_local, 5e5).float()
    ulp = ref.abs().clamp_min(2.0 ** -126) * 2.0 ** -7
    assert bool(((got - ref).abs() <= ulp).all())
    if rows == 1:  # the mean of one row is the row: bit-exact
        assert torch.equal(got, ref)
    assert (got != ref).float().mean().item() < 0.05


@pytest.mark.parametrize("shape", SHAPES, ids=IDS)
@pytest.mark.parametrize("rope_mode", ["ROPE_LLAMA", "NONE"])
def test_sparse_prefill_attention(dev, shape, rope_mode):
    m, S = 77, 413   # ragged tile edges on both axes
    say(f"prefill attention H={shape['num_heads']} Hkv={shape['num_kv_heads']} m={m} S={S} {rope_mode}")
    wl = workloads.build("pf", shape, [S + 50], [64], 1, dev, seed=3, n_init=8, n_local=m)
    c = wl.cfg
    c.rope_mode = rope_mode
    g = torch.Generator(device=dev).manual_seed(4)
    q = torch.randn((m, c.num_heads * 128), generator=g, device=dev).bfloat16()
    sel = wl.table[0, torch.randperm(S + 50, generator=g, device=dev)[:S].long()].contiguous()
    sel_len = torch.tensor([S], dtype=torch.int32, device=dev)
    out = ops.sparse_prefill_attention(c, q, wl.k_pool, wl.v_pool, sel, sel_len)
    torch.cuda.synchronize()
    ref = oracle.prefill.sparse_prefill_attention(q.cpu().view(m, c.num_heads, 128), wl.k_pool.cpu(),
                                                  wl.v_pool.cpu(), sel.cpu(), _sm(c), c.rope_theta,
                                                  c.rope_scale, c.logit_cap, rope_mode)
    err = (out.cpu().float() - ref.reshape(m, -1).float()).abs().max().item()
    assert err <= 2e-2, err


@pytest.mark.parametrize("seed", range(16))
def test_sparse_prefill_attention_randomised(dev, seed):
    """Random chunk sizes, selection lengths and head shapes through the causal attention
    (its key tiles are streamed by four groups of wavefronts that hand buffers to each
    other through counters: every length is another pattern of full, partial and missing
    rounds), with or without the rotation and the soft cap, scaled queries so that the
    running maximum moves.  Within 2e-2 plus two bf16 units of the reference value: the
    rotated keys and the softmax weights enter the matrix products as bf16, which shows
    in outputs above one when doubled queries make the softmax peaked."""
    import random
    rnd = random.Random(4000 + seed)
    shape = SHAPES[rnd.randrange(len(SHAPES))]
    m = rnd.choice([rnd.randrange(1, 17), rnd.randrange(17, 200), rnd.randrange(200, 513)])
    S = m + rnd.choice([0, rnd.randrange(0, 40), rnd.randrange(40, 700), rnd.randrange(700, 2800)])
    rope_mode = rnd.choice(["ROPE_LLAMA", "ROPE_LLAMA", "NONE"])
    cap = rnd.choice([0.0, 0.0, 30.0])
    say(f"prefill attention randomised seed={seed} H={shape['num_heads']} kv={shape['num_kv_heads']} "
        f"m={m} S={S} {rope_mode} cap={cap}")
    wl = workloads.build("pf", shape, [S + 50], [64], 1, dev, seed=4100 + seed, n_init=8, n_local=m)
    c = wl.cfg
    c.rope_mode, c.logit_cap = rope_mode, cap
    g = torch.Generator(device=dev).manual_seed(4200 + seed)
    q = (torch.randn((m, c.num_heads * 128), generator=g, device=dev) * rnd.choice([0.3, 1.0, 2.0])).bfloat16()
    sel = wl.table[0, torch.randperm(S + 50, generator=g, device=dev)[:S].long()].contiguous()
    sel_len = torch.tensor([S], dtype=torch.int32, device=dev)
    out = ops.sparse_prefill_attention(c, q, wl.k_pool, wl.v_pool, sel, sel_len)
    torch.cuda.synchronize()
    ref = oracle.prefill.sparse_prefill_attention(q.cpu().view(m, c.num_heads, 128), wl.k_pool.cpu(),
                                                  wl.v_pool.cpu(), sel.cpu(), _sm(c), c.rope_theta,
                                                  c.rope_scale, c.logit_cap, rope_mode)
    ref = ref.reshape(m, -1).float()
    excess = ((out.cpu().float() - ref).abs() - (2e-2 + 2.0 ** -6 * ref.abs())).max().item()
    assert excess <= 0.0, excess


def test_sparse_prefill_attention_full_chunk_and_soft_cap(dev):
    """A whole 512-row chunk over the selected-list length of the served configs, the
    chunk starting exactly at S - m; and the soft cap."""
    m, S = 512, 2688
    say(f"prefill attention m={m} S={S} (+ soft cap)")
    wl = workloads.build("pf", SHAPES[0], [S], [64], 1, dev, seed=5, n_init=8, n_local=m)
    for cap in (0.0, 30.0):
        c = wl.cfg
        c.logit_cap = cap
        g = torch.Generator(device=dev).manual_seed(6)
        q = (3.0 * torch.randn((m, c.num_heads * 128), generator=g, device=dev)).bfloat16()
        sel = wl.table[0, :S].contiguous()
        sel_len = torch.tensor([S], dtype=torch.int32, device=dev)
        out = ops.sparse_prefill_attention(c, q, wl.k_pool, wl.v_pool, sel, sel_len)
        torch.cuda.synchronize()
        rows = torch.tensor([0, 1, 15, 16, 255, 300, 511])
        ref = oracle.prefill.sparse_prefill_attention(
            q.cpu().view(m, c.num_heads, 128), wl.k_pool.cpu(), wl.v_pool.cpu(), sel.cpu(), _sm(c),
            c.rope_theta, c.rope_scale, cap, c.rope_mode)
        err = (out.cpu().float().view(m, -1)[rows] - ref.reshape(m, -1).float()[rows]).abs().max().item()
        assert err <= 2e-2, (cap, err)


@pytest.mark.parametrize("m,S", [(1, 1), (20, 20), (100, 100), (5, 31), (16, 33), (40, 129), (130, 131)])
def test_sparse_prefill_attention_short_selections(dev, m, S):
    """The first chunk of a request (S = m: every row sees only the chunk up to itself,
    the first rows a single key) and selections shorter than one round of the kernel's
    four tile streams, where some streams have no tile at all."""
    say(f"prefill attention short selection m={m} S={S}")
    wl = workloads.build("pf", SHAPES[0], [S + 8], [8], 1, dev, seed=21, n_init=1, n_local=m)
    c = wl.cfg
    g = torch.Generator(device=dev).manual_seed(22)
    q = torch.randn((m, c.num_heads * 128), generator=g, device=dev).bfloat16()
    sel = wl.table[0, :S].contiguous()
    sel_len = torch.tensor([S], dtype=torch.int32, device=dev)
    out = ops.sparse_prefill_attention(c, q, wl.k_pool, wl.v_pool, sel, sel_len)
    torch.cuda.synchronize()
    ref = oracle.prefill.sparse_prefill_attention(q.cpu().view(m, c.num_heads, 128), wl.k_pool.cpu(),
                                                  wl.v_pool.cpu(), sel.cpu(), _sm(c), c.rope_theta)
    err = (out.cpu().float() - ref.reshape(m, -1).float()).abs().max().item()
    assert err <= 2e-2, err


@pytest.mark.parametrize("direction", ["growing", "shrinking"])
def test_sparse_prefill_attention_moving_maximum(dev, direction):
    """Logits that grow (or fall) steadily along the selected list, by far more than the
    excess at which the kernel raises a row's running maximum: with growing logits every
    round of tiles raises it, with falling ones the first tile's maximum stays and the
    weights of the later keys become tiny."""
    m, S = 48, 700
    say(f"prefill attention with {direction} logits m={m} S={S}")
    wl = workloads.build("pf", SHAPES[0], [S], [8], 1, dev, seed=23, n_init=1, n_local=m)
    c = wl.cfg
    c.rope_mode = "NONE"
    g = torch.Generator(device=dev).manual_seed(24)
    # keys along one direction with a length that moves with the position; values random
    u = torch.ones(128, device=dev)
    ramp = torch.arange(S, device=dev, dtype=torch.float32) * 0.006
    if direction == "shrinking":
        ramp = ramp.flip(0)
    slots = wl.table[0, :S].long()
    k_pool = wl.k_pool.clone()
    k_pool[slots] = (ramp[:, None, None] * u[None, None, :]
                     + 0.05 * torch.randn((S, c.num_kv_heads, 128), generator=g, device=dev)).bfloat16()
    q = (0.5 * u[None, :].repeat(m, c.num_heads)
         + 0.05 * torch.randn((m, c.num_heads * 128), generator=g, device=dev)).bfloat16()
    sel = wl.table[0, :S].contiguous()
    sel_len = torch.tensor([S], dtype=torch.int32, device=dev)
    out = ops.sparse_prefill_attention(c, q, k_pool, wl.v_pool, sel, sel_len)
    torch.cuda.synchronize()
    ref = oracle.prefill.sparse_prefill_attention(q.cpu().view(m, c.num_heads, 128), k_pool.cpu(),
                                                  wl.v_pool.cpu(), sel.cpu(), _sm(c), c.rope_theta,
                                                  rope_mode="NONE")
    # base-2 logits span 0.5 * 0.006 * 128 / sqrt(128) * log2(e) * 700 = 34 over the list
    err = (out.cpu().float() - ref.reshape(m, -1).float()).abs().max().item()
    assert err <= 2e-2, err


def test_sparse_prefill_attention_fewer_keys_than_rows(dev):
    """A selection that reports no keys (one that gave up reports -1) leaves a defined output:
    zeros.  With fewer keys than rows (a chunk longer than the selected list) the first
    rows - S rows sit at negative positions, see nothing and are zero; the others attend to
    their key prefix as the oracle's do."""
    m = 40
    say("prefill attention with fewer keys than rows")
    wl = workloads.build("pf", SHAPES[1], [100], [8], 1, dev, seed=25, n_init=1, n_local=m)
    c = wl.cfg
    g = torch.Generator(device=dev).manual_seed(26)
    q = torch.randn((m, c.num_heads * 128), generator=g, device=dev).bfloat16()
    sel = wl.table[0, :100].contiguous()
    for reported in (-1, 0):
        sel_len = torch.tensor([reported], dtype=torch.int32, device=dev)
        out = ops.sparse_prefill_attention(c, q, wl.k_pool, wl.v_pool, sel, sel_len)
        torch.cuda.synchronize()
        assert torch.count_nonzero(out).item() == 0, reported
    for S, width in ((m - 1, 100), (7, 100), (17, 17), (33, 33)):
        sel_len = torch.tensor([S], dtype=torch.int32, device=dev)
        out = ops.sparse_prefill_attention(c, q, wl.k_pool, wl.v_pool, sel[:width].contiguous(), sel_len)
        torch.cuda.synchronize()
        ref = oracle.prefill.sparse_prefill_attention(q.cpu().view(m, c.num_heads, 128), wl.k_pool.cpu(),
                                                      wl.v_pool.cpu(), sel[:S].cpu(), _sm(c), c.rope_theta)
        assert torch.count_nonzero(out[:m - S]).item() == 0, S
        assert torch.count_nonzero(out[m - S]).item() > 0, S
        assert (out.cpu().float() - ref.reshape(m, -1).float()).abs().max().item() <= 2e-2, S


@pytest.mark.parametrize("rows", [1, 7, 8, 9, 513, 8184, 8200])
def test_kv_store_chunk_sizes(dev, rows):
    """Chunks around the eight rows of a workgroup, a chunk that overflows the table, and
    chunks on both sides of the size up to which the store also writes the length (larger
    ones take a second launch for it)."""
    say(f"kv_store_chunk rows={rows}")
    cfg = ops.LayerConfig(num_heads=4, num_kv_heads=2, n_local=16, top_k=16, rope_theta=1e4)
    g = torch.Generator(device=dev).manual_seed(rows)
    L0, pool_rows = 30, 30 + 8200
    max_tokens = L0 + rows if rows != 513 else L0 + 500      # 513 rows: the last 13 do not fit
    k_pool = torch.zeros((pool_rows, 2, 128), dtype=torch.bfloat16, device=dev)
    v_pool = torch.zeros_like(k_pool)
    k = torch.randn((rows, 2, 128), generator=g, device=dev).bfloat16()
    v = torch.randn((rows, 2, 128), generator=g, device=dev).bfloat16()
    loc = (L0 + torch.randperm(8200, generator=g, device=dev)[:rows]).int()
    table = torch.full((max_tokens,), -1, dtype=torch.int32, device=dev)
    table[:L0] = torch.arange(L0, dtype=torch.int32, device=dev)
    seq = torch.tensor([L0], dtype=torch.int32, device=dev)
    for _ in range(2):      # twice: the length word is left clean for the next call
        seq.fill_(L0)
        ops.kv_store_chunk(cfg, k, v, loc, k_pool, v_pool, table, seq)
        torch.cuda.synchronize()
        kept = min(rows, max_tokens - L0)
        assert int(seq) == L0 + kept
        assert torch.equal(table[L0:L0 + kept], loc[:kept])
        assert torch.equal(k_pool[loc[:kept].long()], k[:kept]) and torch.equal(v_pool[loc[:kept].long()], v[:kept])
        assert torch.equal(table[:L0], torch.arange(L0, dtype=torch.int32, device=dev))


def test_kv_store_chunk(dev):
    say("kv_store_chunk")
    wl = workloads.build("pf", SHAPES[0], [100], [16], 1, dev, seed=7, n_init=4, n_local=16,
                         extra_pages=64)
    c = wl.cfg
    g = torch.Generator(device=dev).manual_seed(8)
    rows = 40
    k = torch.randn((rows, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
    v = torch.randn((rows, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
    loc = (100 + torch.randperm(64, generator=g, device=dev)[:rows]).int()
    table = torch.zeros(200, dtype=torch.int32, device=dev)
    table[:100] = wl.table[0, :100]
    seq = torch.tensor([100], dtype=torch.int32, device=dev)
    ops.kv_store_chunk(c, k, v, loc, wl.k_pool, wl.v_pool, table, seq)
    torch.cuda.synchronize()
    assert int(seq) == 140
    assert torch.equal(table[100:140], loc)
    assert torch.equal(wl.k_pool[loc.long()], k) and torch.equal(wl.v_pool[loc.long()], v)
    assert torch.equal(table[:100], wl.table[0, :100])


@pytest.mark.parametrize("shape", SHAPES[:2], ids=IDS[:2])
@pytest.mark.parametrize("fused", [True, False], ids=["fused", "separate"])
def test_prefill_chunks(dev, shape, fused):
    """Three chunks of an extend forward (the last one ragged) on top of an existing
    context: store, fingerprint, selection, causal attention, chunk by chunk."""
    previous = ops.set_fused_select(fused)
    try:
        L0, T, chunk, top_k = 3000, 150, 64, 96
        say(f"prefill chunks H={shape['num_heads']} L0={L0} T={T} chunk={chunk} fused={fused}")
        wl = workloads.build("pf", shape, [L0], [top_k], 1, dev, seed=11, n_init=8, n_local=chunk,
                             top_k=top_k, extra_pages=T)
        c = wl.cfg
        g = torch.Generator(device=dev).manual_seed(12)
        q = torch.randn((T, c.num_heads * 128), generator=g, device=dev).bfloat16()
        k_new = torch.randn((T, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
        v_new = torch.randn((T, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
        new_slots = (L0 + torch.randperm(T, generator=g, device=dev)).int()
        table = torch.zeros((1, L0 + T), dtype=torch.int32, device=dev)
        table[0, :L0] = wl.table[0, :L0]
        seq = wl.seq_lens_dev.clone()
        layer = ops.PrefillChunk(c, L0 + T, dev, max_rows=chunk)

        kc, vc, tab_cpu = wl.k_pool.cpu(), wl.v_pool.cpu(), table[0].cpu()
        L = L0
        for start in range(0, T, chunk):
            end = min(start + chunk, T)
            m = end - start
            ops.kv_store_chunk(c, k_new[start:end], v_new[start:end], new_slots[start:end].contiguous(),
                               wl.k_pool, wl.v_pool, table[0], seq)
            L += m
            out, sel, sel_pos, sel_len = layer(q[start:end].contiguous(), wl.k_pool, wl.v_pool,
                                               ops.Batch(seq, table, L))
            torch.cuda.synchronize()
            # oracle on the same pools, following the device's fingerprint
            loc = new_slots[start:end].cpu().long()
            kc[loc], vc[loc] = k_new[start:end].cpu(), v_new[start:end].cpu()
            tab_cpu[L - m:L] = new_slots[start:end].cpu()
            qf = ops.fingerprint(c, q[start:end].view(m, c.num_heads, 128).contiguous(),
                                 layer.cos, layer.sin).cpu()
            d = {}
            ref_slots, ref_out = oracle.prefill.prefill_chunk(
                q[start:end].cpu(), kc, vc, tab_cpu, L, c.num_heads, 128, c.n_init, c.n_local, top_k,
                c.rope_theta, c.rope_scale, _sm(c), detail=d, qf_override=qf)
            S = int(sel_len[0])
            assert S == ref_slots.shape[0] == c.n_init + top_k + c.n_local
            pos = sel_pos[0, :S].cpu()
            assert_index_sets_match(pos[c.n_init:c.n_init + top_k], d["top_pos"], d["votes"], c.n_init,
                                    f"chunk at {start}")
            assert pos[-m:].tolist() == list(range(L - m, L))     # the chunk is the tail
            assert torch.equal(sel[0, :S].cpu(), tab_cpu[pos.long()])
            if not torch.equal(sel[0, :S].cpu(), ref_slots):   # a tie went the other way
                ref_out = oracle.prefill.sparse_prefill_attention(
                    q[start:end].cpu().view(m, c.num_heads, 128), kc, vc, sel[0, :S].cpu(), _sm(c),
                    c.rope_theta, c.rope_scale).reshape(m, -1)
            err = (out.cpu().float() - ref_out.float()).abs().max().item()
            assert err <= 2e-2, (start, err)
    finally:
        ops.set_fused_select(previous)


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"H{s['num_heads']}kv{s['num_kv_heads']}")
@pytest.mark.parametrize("chunk", [64, 500])
def test_prefill_step_is_store_then_chunk(dev, shape, chunk):
    """ts_prefill_step (one chunk of the extend forward in one call, tr.py:725-773) against
    ts_kv_store_chunk followed by ts_prefill_chunk, chunk by chunk (the last one ragged, and
    the table full before the end, so that rows are dropped): pools, table, length,
    selections and outputs bit-identical.  The store rides in the fingerprint launch."""
    L0, T, top_k = 3000, 3 * chunk - 17, 96
    say(f"prefill step H={shape['num_heads']} L0={L0} T={T} chunk={chunk}")
    wl = workloads.build("pf", shape, [L0], [top_k], 1, dev, seed=15, n_init=8, n_local=chunk,
                         top_k=top_k, extra_pages=T)
    c = wl.cfg
    g = torch.Generator(device=dev).manual_seed(16)
    q = torch.randn((T, c.num_heads * 128), generator=g, device=dev).bfloat16()
    k_new = torch.randn((T, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
    v_new = torch.randn((T, c.num_kv_heads, 128), generator=g, device=dev).bfloat16()
    new_slots = (L0 + torch.randperm(T, generator=g, device=dev)).int()
    cols = L0 + T - 5                          # the table is full five rows before the end
    results = []
    for one_call in (True, False):
        k_pool, v_pool = wl.k_pool.clone(), wl.v_pool.clone()
        table = torch.zeros((1, cols), dtype=torch.int32, device=dev)
        table[0, :L0] = wl.table[0, :L0]
        seq = wl.seq_lens_dev.clone()
        layer = ops.PrefillChunk(c, cols, dev, max_rows=chunk)
        trace, L = [], L0
        for start in range(0, T, chunk):
            end = min(start + chunk, T)
            L = min(L + end - start, cols)
            bt = ops.Batch(seq, table, L)
            args = (k_new[start:end].contiguous(), v_new[start:end].contiguous(), new_slots[start:end].contiguous())
            if one_call:
                got = layer.step(q[start:end].contiguous(), *args, k_pool, v_pool, bt)
            else:
                ops.kv_store_chunk(c, *args, k_pool, v_pool, table[0], seq)
                got = layer(q[start:end].contiguous(), k_pool, v_pool, bt)
            torch.cuda.synchronize()
            assert not layer.gave_up()
            trace.append([x.clone() for x in got] + [seq.clone(), table.clone()])
        results.append((trace, k_pool, v_pool))
    (ta, ka, va), (tb, kb, vb) = results
    assert torch.equal(ka, kb) and torch.equal(va, vb)
    assert int(ta[-1][4][0]) == cols
    for t, (x, y) in enumerate(zip(ta, tb)):
        assert torch.equal(x[4], y[4]) and torch.equal(x[5], y[5]), f"chunk {t}: length / table"
        assert torch.equal(x[3], y[3]), f"chunk {t}: selection length"
        S = int(x[3][0])
        assert torch.equal(x[1][0, :S], y[1][0, :S]) and torch.equal(x[2][0, :S], y[2][0, :S]), f"chunk {t}"
        assert torch.equal(x[0].view(torch.int16), y[0].view(torch.int16)), f"chunk {t}: output"


def test_prefill_short_context_attends_densely(dev):
    """n_init + k + n_local >= L: the chunk attends over every token so far (tr.py:741-744)."""
    say("prefill chunk, dense context")
    L0, m = 40, 24
    wl = workloads.build("pf", SHAPES[3], [L0 + m], [64], 1, dev, seed=13, n_init=8, n_local=32,
                         top_k=64)
    c = wl.cfg
    g = torch.Generator(device=dev).manual_seed(14)
    q = torch.randn((m, c.num_heads * 128), generator=g, device=dev).bfloat16()
    layer = ops.PrefillChunk(c, L0 + m, dev, max_rows=32)
    out, sel, sel_pos, sel_len = layer(q, wl.k_pool, wl.v_pool, wl.batch)
    torch.cuda.synchronize()
    tab = cpu_tabs(wl)[0]
    assert int(sel_len[0]) == L0 + m
    assert torch.equal(sel[0, :L0 + m].cpu(), tab[:L0 + m])
    ref = oracle.prefill.sparse_prefill_attention(q.cpu().view(m, c.num_heads, 128), wl.k_pool.cpu(),
                                                  wl.v_pool.cpu(), tab[:L0 + m], _sm(c), c.rope_theta)
    assert (out.cpu().float() - ref.reshape(m, -1).float()).abs().max().item() <= 2e-2


@pytest.mark.parametrize("case", ["rows 64, window 16", "the reference's defaults"])
def test_prefill_chunk_longer_than_the_local_window(dev, case):
    """The reference runs any N_Local with its 512-row chunks (its patch() defaults are
    n_init 1, top_k 16, n_local 16): the selected list then ends with the last n_local
    tokens only, the chunk's earlier rows are candidates like any other token, and row i
    sees the entries j <= S - rows + i of the list; with the defaults the list (33 entries)
    is shorter than the chunk, and the rows before the last 33 see nothing."""
    if case == "rows 64, window 16":
        L, m, kw = 500, 64, dict(n_init=4, n_local=16, top_k=96)
    else:
        L, m, kw = 700, 100, dict(n_init=1, n_local=16, top_k=16)
    say(f"prefill chunk beyond the local window: {case}")
    wl = workloads.build("pf", SHAPES[3], [L], [kw["top_k"]], 1, dev, seed=15, **kw)
    c = wl.cfg
    g = torch.Generator(device=dev).manual_seed(16)
    q = torch.randn((m, c.num_heads * 128), generator=g, device=dev).bfloat16()
    layer = ops.PrefillChunk(c, L, dev, max_rows=m)
    out, sel, sel_pos, sel_len = layer(q, wl.k_pool, wl.v_pool, wl.batch)
    torch.cuda.synchronize()
    S = int(sel_len[0])
    assert S == c.n_init + c.top_k + c.n_local
    qf = ops.fingerprint(c, q.view(m, c.num_heads, 128).contiguous(), layer.cos, layer.sin).cpu()
    d = {}
    tab = cpu_tabs(wl)[0]
    ref_slots, ref_out = oracle.prefill.prefill_chunk(
        q.cpu(), wl.k_pool.cpu(), wl.v_pool.cpu(), tab, L, c.num_heads, 128, c.n_init, c.n_local,
        c.top_k, c.rope_theta, c.rope_scale, _sm(c), detail=d, qf_override=qf)
    pos = sel_pos[0, :S].cpu()
    assert_index_sets_match(pos[c.n_init:c.n_init + c.top_k], d["top_pos"], d["votes"], c.n_init, case)
    assert pos[-c.n_local:].tolist() == list(range(L - c.n_local, L))
    assert torch.equal(sel[0, :S].cpu(), tab[pos.long()])
    if not torch.equal(sel[0, :S].cpu(), ref_slots):   # a tie went the other way
        ref_out = oracle.prefill.sparse_prefill_attention(
            q.cpu().view(m, c.num_heads, 128), wl.k_pool.cpu(), wl.v_pool.cpu(), sel[0, :S].cpu(),
            _sm(c), c.rope_theta, c.rope_scale).reshape(m, -1)
    if S < m:
        assert torch.count_nonzero(out[:m - S]).item() == 0
    assert (out.cpu().float() - ref_out.float()).abs().max().item() <= 2e-2
