"""GPU parity of each kernel against the CPU oracle on seeded inputs, through
the C ABI.  Tolerances: fp32 scores 1e-3 relative (to the score RMS); selected
positions identical up to ties at the k-th vote; bf16 attention output 2e-2
absolute."""

import random

import pytest
import torch

import oracle
from tokenselect_amd import ops, workloads
from helpers import (assert_attention_close, assert_index_sets_match, assert_scores_close, cpu_tabs,
                     oracle_layer, say)

pytestmark = pytest.mark.gpu

SHAPES = [
    dict(num_heads=32, num_kv_heads=8, rope_theta=5e5),   # Llama-3-8B
    dict(num_heads=28, num_kv_heads=4, rope_theta=1e6),   # Qwen2-7B
    dict(num_heads=8, num_kv_heads=1, rope_theta=1e4),    # TP shard of a 64/8 model
    dict(num_heads=4, num_kv_heads=2, rope_theta=1e4),
    dict(num_heads=8, num_kv_heads=8, rope_theta=1e4),    # MHA
    dict(num_heads=16, num_kv_heads=4, rope_theta=1e4),
    dict(num_heads=24, num_kv_heads=8, rope_theta=5e5),   # Llama-3.2-3B: three query heads per KV head
    dict(num_heads=12, num_kv_heads=2, rope_theta=1e6),   # Qwen2-1.5B: six
    dict(num_heads=20, num_kv_heads=4, rope_theta=1e4),   # five
]


def small(dev, shape, seed, lens=(3000,), ks=(64,), page=1, n_init=8, n_local=16, **kw):
    return workloads.build("small", shape, list(lens), list(ks), page, dev, seed,
                           n_init=n_init, n_local=n_local, **kw)


def fingerprint(wl, dev):
    c = wl.cfg
    cos, sin = ops.scoring_cos_sin(c.head_dim, c.rope_theta, c.rope_scale, c.n_local, dev)
    return ops.rope_apply(wl.q.view(len(wl.seq_lens), c.num_heads, c.head_dim), cos, sin, None)


def test_rope_apply_bit_exact(dev):
    say("rope_apply rows=5 heads=6 dim=128")
    torch.manual_seed(0)
    x = torch.randn(5, 6, 128).bfloat16()
    pos = torch.tensor([0, 3, 511, 512, 77])
    cos, sin = oracle.rope.cos_sin_tables(513, 128, 5e5, 1.0)
    ref = oracle.rope.apply(x, pos, 5e5, 1.0)
    got = ops.rope_apply(x.to(dev), cos.squeeze(1).contiguous().to(dev),
                         sin.squeeze(1).contiguous().to(dev), pos.to(dev))
    assert torch.equal(got.cpu().view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"H{s['num_heads']}kv{s['num_kv_heads']}")
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_paged_matmul(dev, shape, out_dtype):
    H, Hkv = shape["num_heads"], shape["num_kv_heads"]
    say(f"paged_matmul H={H} Hkv={Hkv} n=2500 out={out_dtype}")
    g = torch.Generator().manual_seed(H * 100 + Hkv)
    P, n = 4096, 2500
    token = torch.randn(P, Hkv, 128, generator=g).bfloat16()
    query = torch.randn(H, 128, generator=g).bfloat16()
    idx = torch.randperm(P, generator=g)[:n].int()
    scores = torch.empty((H, n), dtype=out_dtype, device=dev)
    ops.paged_matmul(query.to(dev), token.to(dev), idx.to(dev), scores, n, H, Hkv, 128)
    ref = oracle.select.score(query, token, idx)
    if out_dtype == torch.float32:
        assert_scores_close(scores.cpu(), ref, "paged_matmul fp32")
    else:  # one bf16 rounding of the fp32 score: within one bf16 ulp (2^-8 relative)
        got = scores.float().cpu()
        assert bool(((got - ref).abs() <= ref.abs() * 2.0 ** -8 + 1e-6).all())
        assert (got != ref.bfloat16().float()).float().mean().item() < 1e-3


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"H{s['num_heads']}kv{s['num_kv_heads']}")
@pytest.mark.parametrize("page", [1, 16])
def test_score_vote_topk(dev, shape, page):
    lens, ks = [3000, 777, 40, 1531], [64, 100, 64, 1]
    say(f"score/vote/topk H={shape['num_heads']} Hkv={shape['num_kv_heads']} page={page} lens={lens}")
    wl = small(dev, shape, seed=page + shape["num_heads"], lens=lens, ks=ks, page=page, top_k=100)
    c = wl.cfg
    qf = fingerprint(wl, dev)
    scores, partials = ops.score(c, wl.batch, qf, wl.k_pool)
    votes, stats = ops.vote(c, wl.batch, scores, partials)
    sel, sel_pos, sel_len = ops.topk_ragged(c, wl.batch, votes)
    torch.cuda.synchronize()
    details = []
    ref_sel, _ = oracle_layer(wl, details)
    tabs = cpu_tabs(wl)
    for b, (L, k) in enumerate(zip(wl.seq_lens, wl.k_list)):
        S = int(sel_len[b])
        if oracle.select.is_dense(L, c.n_init, c.n_local, k):
            assert S == L
            assert torch.equal(sel[b, :L].cpu(), tabs[b][:L])
            assert torch.equal(sel_pos[b, :L].cpu(), torch.arange(L, dtype=torch.int32))
            continue
        d = details[b]
        n = L - c.n_init - c.n_local
        assert torch.equal(qf[b].reshape(-1).cpu().view(torch.int16), d["qf"].view(torch.int16))
        assert_scores_close(ops.scores_head_major(c, scores)[b, :, :n].cpu(), d["scores"],
                            f"scores b={b}")
        ref_stats_m = d["scores"].max(dim=1).values
        assert torch.allclose(stats[b, :, 0].cpu(), ref_stats_m, rtol=1e-5, atol=1e-5)
        assert torch.allclose(votes[b, :n].cpu(), d["votes"], rtol=2e-4, atol=1e-9)
        assert S == c.n_init + k + c.n_local
        pos = sel_pos[b, :S].cpu()
        assert torch.equal(pos[:c.n_init], torch.arange(c.n_init, dtype=torch.int32))
        assert torch.equal(pos[c.n_init + k:], torch.arange(L - c.n_local, L, dtype=torch.int32))
        mid = pos[c.n_init:c.n_init + k]
        assert bool((mid[1:] > mid[:-1]).all()) if k > 1 else True
        assert_index_sets_match(mid, d["top_pos"], d["votes"], c.n_init, f"top-k b={b}")
        assert torch.equal(sel[b, :S].cpu(), tabs[b][pos.long()])


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"H{s['num_heads']}kv{s['num_kv_heads']}")
@pytest.mark.parametrize("page", [1, 16])
def test_fused_select(dev, shape, page):
    """The single-launch selection against the oracle's votes and selection and against
    the separate kernels, twice in a row on one workspace (its counters are
    accumulated into, so a missed clearing shows up on the second pass)."""
    lens, ks = [3000, 777, 40, 1531], [64, 100, 64, 1]
    say(f"fused select H={shape['num_heads']} Hkv={shape['num_kv_heads']} page={page} lens={lens}")
    wl = small(dev, shape, seed=page + shape["num_heads"], lens=lens, ks=ks, page=page, top_k=100)
    c = wl.cfg
    assert ops.select_supported(c, len(lens), max(lens))
    qf = fingerprint(wl, dev)
    details = []
    oracle_layer(wl, details)
    votes_sep, _ = ops.vote(c, wl.batch, *ops.score(c, wl.batch, qf, wl.k_pool))
    sel_sep, pos_sep, len_sep = ops.topk_ragged(c, wl.batch, votes_sep)
    space = None
    for attempt in range(2):
        sel, sel_pos, sel_len, votes, space = ops.select(c, wl.batch, qf, wl.k_pool,
                                                         want_votes=True, workspace=space)
        torch.cuda.synchronize()
        assert not ops.select_fault(c, wl.batch, space)
        assert torch.equal(sel_len, len_sep)
        tabs = cpu_tabs(wl)
        for b, (L, k) in enumerate(zip(wl.seq_lens, wl.k_list)):
            S = int(sel_len[b])
            if not details[b]:  # dense
                assert torch.equal(sel[b, :S], sel_sep[b, :S])
                assert torch.equal(sel_pos[b, :S], pos_sep[b, :S])
                continue
            n = L - c.n_init - c.n_local
            assert torch.allclose(votes[b, :n].cpu(), details[b]["votes"], rtol=2e-4, atol=1e-9), \
                f"votes b={b} attempt={attempt}"
            pos = sel_pos[b, :S].cpu()
            mid = pos[c.n_init:c.n_init + k]
            assert bool((mid[1:] > mid[:-1]).all()) if k > 1 else True
            assert_index_sets_match(mid, details[b]["top_pos"], details[b]["votes"], c.n_init,
                                    f"fused top-k b={b} attempt={attempt}")
            assert torch.equal(pos[:c.n_init], pos_sep[b, :c.n_init].cpu())
            assert torch.equal(pos[c.n_init + k:], pos_sep[b, c.n_init + k:S].cpu())
            assert torch.equal(sel[b, :S].cpu(), tabs[b][pos.long()])


@pytest.mark.parametrize("lens", [[5000, 3000, 9000], [40000, 20000]], ids=["3x<=9K", "2x<=40K"])
def test_fused_select_same_with_either_workgroup_size(dev, lens):
    """A batch whose scores fit one workgroup per CU is served that way, unless requests
    may be skipped (hit flags given), which puts it on two smaller workgroups per CU: the
    same inputs through both, alternating on one workspace, must give the same votes up
    to the rounding of the merged statistics (the chunks they are merged from differ:
    2e-6 relative) and the same selection; the votes are also held against the oracle's."""
    say(f"fused select, one and two workgroups per CU, lens={lens}")
    ks = [256] * len(lens)
    wl = small(dev, SHAPES[0], seed=len(lens), lens=lens, ks=ks, page=16, top_k=256)
    c = wl.cfg
    qf = fingerprint(wl, dev)
    details = []
    oracle_layer(wl, details)
    nobody = torch.zeros(len(lens), dtype=torch.int32, device=dev)  # hit flags: every request misses
    cache = ops.SelectionCache.allocate(c, len(lens), dev)
    space = None
    results = []
    for attempt in range(4):
        skipping = dict(hit=nobody, cache=cache) if attempt % 2 else {}
        sel, sel_pos, sel_len, votes, space = ops.select(c, wl.batch, qf, wl.k_pool, want_votes=True,
                                                         workspace=space, **skipping)
        torch.cuda.synchronize()
        assert not ops.select_fault(c, wl.batch, space)
        results.append((sel.clone(), sel_pos.clone(), sel_len.clone(), votes.clone()))
    first = results[0]
    for attempt, got in enumerate(results[1:], 1):
        assert torch.equal(got[2], first[2]), f"attempt {attempt}: lengths"
        for b, (L, k) in enumerate(zip(lens, ks)):
            S, n = int(first[2][b]), L - c.n_init - c.n_local
            assert torch.allclose(got[3][b, :n], first[3][b, :n], rtol=2e-6, atol=0), f"attempt {attempt} b={b}: votes"
            mid = got[1][b, c.n_init:c.n_init + k].cpu()
            assert_index_sets_match(mid, first[1][b, c.n_init:c.n_init + k].cpu(), first[3][b, :n].cpu(),
                                    c.n_init, f"attempt {attempt} b={b}")
            assert torch.equal(got[0][b, :S].cpu(), cpu_tabs(wl)[b][got[1][b, :S].cpu().long()])
    for b, L in enumerate(lens):
        n = L - c.n_init - c.n_local
        assert torch.allclose(first[3][b, :n].cpu(), details[b]["votes"], rtol=2e-4, atol=1e-9), f"votes b={b}"
        assert_index_sets_match(first[1][b, c.n_init:c.n_init + ks[b]].cpu(), details[b]["top_pos"],
                                details[b]["votes"], c.n_init, f"oracle b={b}")


def test_select_clear_then_cleared_equals_select(dev):
    """ts_select is ts_select_clear + ts_select_cleared: the two calls made by hand,
    twice in a row on one workspace, give what the single call gives."""
    say("select_clear + select(cleared) against select")
    lens, ks = [3000, 777, 40, 1531], [64, 100, 64, 1]
    wl = small(dev, SHAPES[0], seed=5, lens=lens, ks=ks, page=16, top_k=100)
    c = wl.cfg
    qf = fingerprint(wl, dev)
    want = ops.select(c, wl.batch, qf, wl.k_pool, want_votes=True)
    space = ops.select_workspace(c, wl.batch, dev)
    for attempt in range(2):
        ops.select_clear(c, wl.batch, space)
        got = ops.select(c, wl.batch, qf, wl.k_pool, want_votes=True, workspace=space, cleared=True)
        torch.cuda.synchronize()
        assert not ops.select_fault(c, wl.batch, space)
        assert torch.equal(got[2], want[2])
        for b, L in enumerate(lens):
            S = int(want[2][b])
            assert torch.equal(got[0][b, :S], want[0][b, :S]) and torch.equal(got[1][b, :S], want[1][b, :S])
            n = L - c.n_init - c.n_local
            if n > 0 and S < L:
                assert torch.equal(got[3][b, :n], want[3][b, :n])
    with pytest.raises(ValueError, match="cleared"):
        ops.select(c, wl.batch, qf, wl.k_pool, cleared=True)


def test_fused_select_ties(dev):
    """Duplicated key rows give exactly equal votes: the k-th vote is shared by many
    candidates and the ones at the lowest positions must win, as in the separate
    top-k; the cut falls in the middle of a workgroup and between workgroups."""
    say("fused select: exact ties at the k-th vote")
    for seed, (L, k) in enumerate([(4000, 300), (4000, 64), (1500, 700)]):
        wl = small(dev, SHAPES[0], seed=50 + seed, lens=[L], ks=[k], page=1, top_k=k)
        c = wl.cfg
        # Every candidate row becomes a copy of one of 7 rows: 7 distinct votes.
        tab = wl.table[0, :L].long()
        src = tab[c.n_init + (torch.arange(L, device=dev) % 7)]
        wl.k_pool[tab] = wl.k_pool[src]
        qf = fingerprint(wl, dev)
        votes_sep, _ = ops.vote(c, wl.batch, *ops.score(c, wl.batch, qf, wl.k_pool))
        _, pos_sep, len_sep = ops.topk_ragged(c, wl.batch, votes_sep)
        _, sel_pos, sel_len, votes, space = ops.select(c, wl.batch, qf, wl.k_pool, want_votes=True)
        torch.cuda.synchronize()
        assert not ops.select_fault(c, wl.batch, space)
        n = L - c.n_init - c.n_local
        assert torch.unique(votes[0, :n]).numel() <= 7
        assert torch.allclose(votes[0, :n], votes_sep[0, :n], rtol=1e-5, atol=0)
        assert torch.equal(sel_len, len_sep)
        assert torch.equal(sel_pos[0, :int(sel_len[0])], pos_sep[0, :int(sel_len[0])])


@pytest.mark.parametrize("fused_select", [True, False], indirect=True, ids=["fused", "separate"])
def test_select_with_all_votes_equal(dev, fused_select):
    """A zero query makes every vote H/n: one histogram bin at every level, every
    candidate tied at the k-th vote; the k lowest positions win.  (Also a guard against
    the selection serialising on one counter: the layer must not take milliseconds.)"""
    say(f"selection with all votes equal, fused={fused_select}")
    L, k = 70000, 1000
    wl = small(dev, SHAPES[0], seed=81, lens=[L], ks=[k], page=16, top_k=k, n_init=128, n_local=512)
    wl.q.zero_()
    c = wl.cfg
    layer = ops.DecodeLayer(c, 1, L, dev)
    layer(wl.q, wl.k_pool, wl.v_pool, wl.batch)
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    out, sel, sel_pos, sel_len = layer(wl.q, wl.k_pool, wl.v_pool, wl.batch)
    end.record()
    torch.cuda.synchronize()
    S = int(sel_len[0])
    assert S == c.n_init + k + c.n_local
    expect = torch.cat([torch.arange(c.n_init + k), torch.arange(L - c.n_local, L)]).int()
    assert torch.equal(sel_pos[0, :S].cpu(), expect)
    assert start.elapsed_time(end) < 1.0, "the selection serialised on a single counter"


def test_fused_select_reports_a_wait_that_gave_up(dev):
    """The give-up path, forced from the host so that every kernel still exits normally: one
    team member that never arrives and a 20 us bound.  Every wait runs into the bound, the
    kernel drains, and the launch says so without a synchronisation of its own: sel_len = -1
    for the selecting requests, the caller's word, the word in the workspace.  The next
    launch on the same workspace is correct."""
    import time
    lens, ks = [3000, 40, 1531], [64, 64, 100]
    say(f"fused select, forced give-up lens={lens}")
    wl = small(dev, SHAPES[0], seed=77, lens=lens, ks=ks, page=16, top_k=100)
    c = wl.cfg
    qf = fingerprint(wl, dev)
    word = ops.fault_word()
    bt = ops.Batch(wl.batch.seq_lens, wl.batch.table, wl.batch.max_seq_len, wl.batch.k_per_req, word)
    space = ops.select_workspace(c, bt, dev)
    torch.cuda.synchronize()
    t0 = time.time()
    sel, sel_pos, sel_len, _, _ = ops.select(c, bt, qf, wl.k_pool, workspace=space, wait_ticks=2000,
                                             absent_workgroups=1)
    torch.cuda.synchronize()
    assert time.time() - t0 < 1.0, "a wait that gave up must not be waited for again"
    assert sel_len.tolist() == [-1, 40, -1]          # the dense request needs no rendezvous
    assert torch.equal(sel[1, :40].cpu(), cpu_tabs(wl)[1][:40])
    assert int(word[0]) == 1 and ops.select_fault(c, bt, space)
    with pytest.raises(ops.SelectionGaveUp):
        ops.raise_if_gave_up(word)
    # an attention over the reported lengths reads nothing of the invalid lists
    out = ops.sparse_decode_attention(c, wl.q, wl.k_pool, wl.v_pool, sel, sel_len)
    torch.cuda.synchronize()
    assert out.shape[0] == 3
    # the same workspace, cleared by the next call: the selection of the separate kernels
    word.zero_()
    votes_sep, _ = ops.vote(c, bt, *ops.score(c, bt, qf, wl.k_pool))
    sel_sep, pos_sep, len_sep = ops.topk_ragged(c, bt, votes_sep)
    sel, sel_pos, sel_len, _, _ = ops.select(c, bt, qf, wl.k_pool, workspace=space)
    torch.cuda.synchronize()
    assert int(word[0]) == 0 and not ops.select_fault(c, bt, space)
    assert torch.equal(sel_len, len_sep)
    for b in range(3):
        S = int(sel_len[b])
        assert torch.equal(sel[b, :S], sel_sep[b, :S]) and torch.equal(sel_pos[b, :S], pos_sep[b, :S])


def layer_matches_oracle(wl, out, sel, sel_pos, sel_len, tag):
    details = []
    ref_sel, ref_out = oracle_layer(wl, details)
    c = wl.cfg
    for b in range(len(wl.seq_lens)):
        S = int(sel_len[b])
        assert S == ref_sel[b].shape[0], f"{tag} b={b}: {S} slots, oracle {ref_sel[b].shape[0]}"
        if details[b]:
            assert_index_sets_match(sel_pos[b, c.n_init:S - c.n_local].cpu(), details[b]["top_pos"],
                                    details[b]["votes"], c.n_init, f"{tag} top-k b={b}")
        assert_attention_close(wl, b, out[b], sel[b, :S], ref_sel[b], ref_out[b], f"{tag} b={b}")


def test_layer_object_recovers_a_step_that_gave_up(dev):
    """A decode layer whose selection gives up (forced from the host: one team member that
    never arrives, a 20 us bound; every kernel exits normally) reports it in its pinned word;
    recover() at the caller's synchronisation point repeats the step's selection and
    attention with the separate kernels and returns the oracle's output, and the object
    stays on the separate kernels.  A give-up that nobody recovered makes the next call
    switch over and raise, after which the object works."""
    import dataclasses
    lens, ks = [3000, 40, 1531], [64, 64, 100]
    say(f"decode layer, forced give-up and recovery lens={lens}")
    wl = small(dev, SHAPES[0], seed=78, lens=lens, ks=ks, page=16, top_k=100)
    forced = dataclasses.replace(wl.batch, wait_us=20, absent_workgroups=1)
    layer = ops.DecodeLayer(wl.cfg, 3, max(lens), dev)
    assert ops.layer_selection_form(wl.cfg, wl.batch) == 2
    out, sel, sel_pos, sel_len = layer(wl.q, wl.k_pool, wl.v_pool, forced)
    torch.cuda.synchronize()
    assert layer.gave_up() and sel_len.tolist() == [-1, 40, -1]
    got = layer.recover(wl.q, wl.k_pool, wl.v_pool, forced)
    assert got is not None and layer.separate and not layer.gave_up()
    torch.cuda.synchronize()
    layer_matches_oracle(wl, *got, "recovered step")
    # nothing to recover now, and the object no longer launches kernels that could give up
    assert layer.recover(wl.q, wl.k_pool, wl.v_pool, forced) is None
    again = layer(wl.q, wl.k_pool, wl.v_pool, forced)
    torch.cuda.synchronize()
    assert not layer.gave_up()
    layer_matches_oracle(wl, *again, "after the switch")
    # a give-up that nobody recovered: the next call switches over and raises, then works
    other = ops.DecodeLayer(wl.cfg, 3, max(lens), dev)
    other(wl.q, wl.k_pool, wl.v_pool, forced)
    torch.cuda.synchronize()
    with pytest.raises(ops.SelectionGaveUp):
        other(wl.q, wl.k_pool, wl.v_pool, wl.batch)
    assert other.separate and not other.gave_up()
    retried = other(wl.q, wl.k_pool, wl.v_pool, wl.batch)
    torch.cuda.synchronize()
    layer_matches_oracle(wl, *retried, "retried step")
    # one call on the separate kernels without touching the process-wide switch
    third = ops.DecodeLayer(wl.cfg, 3, max(lens), dev)
    once = third(wl.q, wl.k_pool, wl.v_pool, dataclasses.replace(forced, separate_kernels=True))
    torch.cuda.synchronize()
    assert not third.gave_up() and not third.separate
    layer_matches_oracle(wl, *once, "separate kernels for one call")


def test_recovery_keeps_the_selection_cache_consistent(dev):
    """Selection-cache trace in which one step gives up (forced) and is recovered: the requests
    that were selecting select afresh, those that hit keep their cached positions, the counters
    advance once per step, and every later decision equals that of an undisturbed run."""
    import dataclasses
    B, steps, bad = 3, 8, 4
    lens = [2500, 3000, 2800]
    say(f"selection cache trace with a recovered give-up at step {bad}")
    wl = small(dev, SHAPES[0], seed=91, lens=lens, ks=[64] * B, page=1, top_k=64)
    c = wl.cfg
    g = torch.Generator().manual_seed(92)
    qs = [wl.q.cpu().float()]
    for t in range(1, steps):   # request 0 drifts slowly (hits), 1 jumps (misses), 2 alternates
        fresh = torch.randn(qs[0].shape, generator=g)
        mix = torch.tensor([0.99, 0.0, 0.99 if t % 2 else 0.0])[:, None]
        qs.append(mix * qs[-1] + (1 - mix ** 2).sqrt() * fresh)
    qs = [q.bfloat16().to(dev) for q in qs]

    def run(disturb):
        cache = ops.SelectionCache.allocate(c, B, dev)
        layer = ops.DecodeLayer(c, B, max(lens), dev)
        trace = []
        for t in range(steps):
            bt = wl.batch
            if disturb and t == bad:
                bt = dataclasses.replace(bt, wait_us=20, absent_workgroups=1)
            res = layer(qs[t], wl.k_pool, wl.v_pool, bt, cache)
            if disturb:
                got = layer.recover(qs[t], wl.k_pool, wl.v_pool, bt, cache)
                assert (got is not None) == (t == bad)
                res = got or res
            torch.cuda.synchronize()
            trace.append([x.clone() for x in res] + [cache.counters.clone(), cache.cache_len.clone(),
                                                       cache.topk_cache.clone()])
        return trace

    plain, disturbed = run(False), run(True)
    for t in range(steps):
        for name, x, y in zip(("out", "sel", "sel_pos", "sel_len", "counters", "cache_len", "topk_cache"),
                              plain[t], disturbed[t]):
            if name == "out":
                assert (x.float() - y.float()).abs().max().item() <= 2e-2, f"step {t}"
            else:
                assert torch.equal(x, y), f"step {t}: {name} differs after the recovery"
    hits = plain[-1][4][:, 0].tolist()
    assert hits[0] >= steps - 2 and hits[1] == 0, f"the trace should mix hits and misses: {hits}"


def test_fused_select_rejects_unsupported(dev):
    say("fused select: pool_kernel above 256 -> TS_ESHAPE")
    wl = small(dev, SHAPES[0], seed=3, lens=[2000], ks=[64], pool_kernel=300)
    assert not ops.select_supported(wl.cfg, 1, 2000)
    with pytest.raises(RuntimeError, match="ts_select"):
        ops.select(wl.cfg, wl.batch, fingerprint(wl, dev), wl.k_pool)


@pytest.mark.parametrize("kernel", [5, 6, 32, 128, 255])
@pytest.mark.parametrize("page", [1, 16])
def test_fused_select_max_pool(dev, kernel, page):
    """Max-pooled votes inside the single-launch selection (the neighbours' votes cross
    workgroup borders): against the oracle, and exact on the kernel's own pooled votes,
    where runs of equal values make ties at the k-th vote the rule."""
    lens, ks = [3000, 777, 40, 1531], [64, 100, 64, 17]
    say(f"fused select with max-pool kernel={kernel} page={page}")
    wl = small(dev, SHAPES[0], seed=60 + kernel, lens=lens, ks=ks, page=page, top_k=100,
               pool_kernel=kernel)
    c = wl.cfg
    assert ops.select_supported(c, len(lens), max(lens))
    qf = fingerprint(wl, dev)
    details = []
    oracle_layer(wl, details)
    space = None
    for attempt in range(2):
        sel, sel_pos, sel_len, votes, space = ops.select(c, wl.batch, qf, wl.k_pool,
                                                         want_votes=True, workspace=space)
        torch.cuda.synchronize()
        assert not ops.select_fault(c, wl.batch, space)
        for b, (L, k) in enumerate(zip(wl.seq_lens, wl.k_list)):
            S = int(sel_len[b])
            if not details[b]:  # dense
                assert S == L
                continue
            n_out = details[b]["votes"].shape[0]
            assert n_out == L - c.n_init - c.n_local - (1 if kernel % 2 == 0 else 0)
            v = votes[b, :n_out]
            assert torch.allclose(v.cpu(), details[b]["votes"], rtol=2e-4, atol=1e-9), \
                f"pooled votes b={b} attempt={attempt}"
            mid = sel_pos[b, c.n_init:c.n_init + k].long()
            assert S == c.n_init + k + c.n_local
            assert bool((mid[1:] > mid[:-1]).all())
            assert_index_sets_match(mid.cpu(), details[b]["top_pos"], details[b]["votes"], c.n_init,
                                    f"fused pooled top-k b={b} attempt={attempt}", rtol=3e-4)
            chosen = torch.zeros(n_out, dtype=torch.bool, device=dev)
            chosen[mid - c.n_init] = True
            lowest_in, highest_out = v[chosen].min(), v[~chosen].max()
            assert float(lowest_in) >= float(highest_out)
            tied_in = torch.nonzero(chosen & (v == lowest_in)).flatten()
            tied_out = torch.nonzero(~chosen & (v == lowest_in)).flatten()
            if tied_out.numel():
                assert int(tied_in.max()) < int(tied_out.min()), f"tie order b={b}"


@pytest.mark.parametrize("case", ["wide", "narrow", "tie_groups_small", "tie_groups_large"])
def test_fused_select_every_resolution_path(dev, case):
    """The single-launch selection resolves the k-th vote by histogram levels until the
    threshold bin holds at most 256 candidates, which it then lists and ranks: a
    heavy-tailed vote distribution lists after the first level, a narrow one (tiny
    query) after the second, many exact ties (keys drawn from a few distinct rows) go
    through all three levels and the count of ties.  Checked exactly on the kernel's
    own votes: no unselected vote above a selected one, ties lowest position first."""
    say(f"fused select resolution path: {case}")
    L, k = 60000, 1000
    wl = small(dev, SHAPES[0], seed=90, lens=[L, 9000], ks=[k, 300], page=16, top_k=k, n_init=128,
               n_local=512)
    c = wl.cfg
    g = torch.Generator(device=dev).manual_seed(91)
    if case == "narrow":
        wl.q.mul_(0.02)
    if case.startswith("tie_groups"):
        groups = 400 if case == "tie_groups_small" else 3
        distinct = torch.randn(groups, c.num_kv_heads, c.head_dim, device=dev, generator=g).bfloat16()
        which = torch.randint(groups, (wl.k_pool.shape[0],), device=dev, generator=g)
        wl.k_pool.copy_(distinct[which])
    qf = fingerprint(wl, dev)
    space = None
    for attempt in range(2):
        sel, sel_pos, sel_len, votes, space = ops.select(c, wl.batch, qf, wl.k_pool,
                                                         want_votes=True, workspace=space)
        torch.cuda.synchronize()
        assert not ops.select_fault(c, wl.batch, space)
        for b, (Lb, kb) in enumerate(zip(wl.seq_lens, wl.k_list)):
            n = Lb - c.n_init - c.n_local
            assert int(sel_len[b]) == c.n_init + kb + c.n_local
            v = votes[b, :n]
            mid = sel_pos[b, c.n_init:c.n_init + kb].long()
            assert bool((mid[1:] > mid[:-1]).all()), f"{case} b={b}: not ascending"
            assert int(mid.min()) >= c.n_init and int(mid.max()) < Lb - c.n_local
            chosen = torch.zeros(n, dtype=torch.bool, device=dev)
            chosen[mid - c.n_init] = True
            lowest_in, highest_out = v[chosen].min(), v[~chosen].max()
            assert float(lowest_in) >= float(highest_out), f"{case} b={b} attempt={attempt}"
            tied_in = torch.nonzero(chosen & (v == lowest_in)).flatten()
            tied_out = torch.nonzero(~chosen & (v == lowest_in)).flatten()
            if tied_out.numel():
                assert int(tied_in.max()) < int(tied_out.min()), f"{case} b={b}: tie order"
            # the table translation of the selected positions
            slots = wl.batch.table[b].long()[mid // c.page_size] * c.page_size + mid % c.page_size
            assert torch.equal(sel[b, c.n_init:c.n_init + kb].long(), slots)
        # the case is in the regime it is meant to exercise (request 0)
        keys = votes[0, :L - 640].view(torch.int32).long() | (1 << 31)
        kth = keys.sort(descending=True).values[k - 1]
        in_bin = {bits: int(((keys >> (32 - bits)) == (kth >> (32 - bits))).sum()) for bits in (11, 22)}
        if case == "wide":
            assert in_bin[11] <= 256, in_bin
        elif case == "tie_groups_large":
            assert in_bin[22] > 256, in_bin
        else:
            assert in_bin[11] > 256 >= in_bin[22], in_bin
    # same inputs through the separate kernels: identical positions
    scores, partials = ops.score(c, wl.batch, qf, wl.k_pool)
    votes_sep, _ = ops.vote(c, wl.batch, scores, partials)
    _, pos_sep, len_sep = ops.topk_ragged(c, wl.batch, votes_sep)
    assert torch.equal(len_sep, sel_len)
    for b, Lb in enumerate(wl.seq_lens):
        n = Lb - c.n_init - c.n_local
        if torch.equal(votes_sep[b, :n], votes[b, :n]):
            assert torch.equal(pos_sep[b, :int(len_sep[b])], sel_pos[b, :int(sel_len[b])])


def test_select_randomised(dev):
    """Both forms of the selection (single launch; score + vote + ragged top-k).  Seeded sweep over shapes, ragged batches, page sizes, sink / local sizes, k (zero
    included), max-pool windows and vote distributions (heavy-tailed, nearly uniform,
    tie groups of about 256 = the capacity of the short candidate list, all equal):
    the middle segment is exactly the k best of the kernel's own votes, ties lowest
    position first; the sink, the local window and the slot translation are exact."""
    import random
    for seed in range(60):
        rnd = random.Random(1000 + seed)
        shape = rnd.choice(SHAPES)
        B = rnd.choice([1, 1, 2, 3, 5])
        lens = [rnd.randint(30, 40000 if seed % 4 == 0 else 6000) for _ in range(B)]
        top_k = rnd.choice([1, 17, 100, 256, 1000, 2048])
        ks = [rnd.randint(0, top_k) if rnd.random() < 0.2 else top_k for _ in range(B)]
        page = rnd.choice([1, 16])
        n_init, n_local = rnd.choice([(0, 1), (8, 16), (128, 512)])
        pool = rnd.choice([-1, -1, 5, 6, 32])
        mode = rnd.choice(["wide", "narrow", "ties", "ties256", "zero"])
        say(f"randomised select seed={seed} H={shape['num_heads']}/{shape['num_kv_heads']} lens={lens} "
            f"ks={ks} page={page} sink/local={n_init}/{n_local} pool={pool} votes={mode}")
        wl = small(dev, shape, seed=seed, lens=lens, ks=ks, page=page, n_init=n_init, n_local=n_local,
                   top_k=top_k, pool_kernel=pool)
        c = wl.cfg
        if not ops.select_supported(c, B, max(lens)):
            continue
        g = torch.Generator(device=dev).manual_seed(seed)
        if mode == "narrow":
            wl.q.mul_(rnd.choice([0.02, 0.1]))
        elif mode == "wide" and B > 1:
            # a scale per request: the requests of one launch then need different numbers
            # of histogram levels
            scale = torch.tensor([rnd.choice([1.0, 0.02, 0.2, 0.0]) for _ in range(B)], device=dev)
            wl.q.copy_((wl.q.view(B, -1).float() * scale.view(B, 1)).to(wl.q.dtype).view(wl.q.shape))
        elif mode == "zero":
            wl.q.zero_()
        elif mode in ("ties", "ties256"):
            n0 = max(lens[0] - n_init - n_local, 1)
            groups = (max(1, n0 // rnd.choice([250, 256, 257, 300])) if mode == "ties256"
                      else rnd.choice([2, 7, 40, 400]))
            distinct = torch.randn(groups, c.num_kv_heads, c.head_dim, device=dev, generator=g).bfloat16()
            which = torch.randint(groups, (wl.k_pool.shape[0],), device=dev, generator=g)
            wl.k_pool.copy_(distinct[which])
        qf = fingerprint(wl, dev)
        sel, sel_pos, sel_len, votes, space = ops.select(c, wl.batch, qf, wl.k_pool, want_votes=True)
        torch.cuda.synchronize()
        assert not ops.select_fault(c, wl.batch, space)
        votes_sep, _ = ops.vote(c, wl.batch, *ops.score(c, wl.batch, qf, wl.k_pool))
        separate = ops.topk_ragged(c, wl.batch, votes_sep)
        # The same launch with threshold hints: none yet, its own from the launch before, then
        # hints moved by a few bins or set to nonsense, request by request.  Bit for bit the same.
        import dataclasses
        hint = torch.zeros(B, dtype=torch.int32, device=dev)
        hinted = dataclasses.replace(wl.batch, hint=hint)
        for launch in range(4):
            if launch >= 2:
                moved = [rnd.choice([-5, -3, -1, 0, 1, 2, 4, 6, 900, -10000]) for _ in range(B)]
                hint.add_(torch.tensor(moved, dtype=torch.int32, device=dev))
            got = ops.select(c, hinted, qf, wl.k_pool, workspace=space)
            torch.cuda.synchronize()
            assert not ops.select_fault(c, hinted, space), f"seed={seed} launch {launch}"
            assert torch.equal(got[2], sel_len), f"seed={seed} launch {launch}: lengths"
            for b in range(B):
                S = int(sel_len[b])
                assert torch.equal(got[0][b, :S], sel[b, :S]) and torch.equal(got[1][b, :S], sel_pos[b, :S]), \
                    f"seed={seed} launch {launch} b={b}: the selection with a hint differs"
        for path, (sel, sel_pos, sel_len), votes in (("fused", (sel, sel_pos, sel_len), votes),
                                                     ("separate", separate, votes_sep)):
            for b, (L, k) in enumerate(zip(lens, ks)):
                what = f"seed={seed} b={b} {path}"
                S = int(sel_len[b])
                if n_init + k + n_local >= L:
                    assert S == L and torch.equal(sel_pos[b, :L].cpu(), torch.arange(L, dtype=torch.int32))
                    continue
                n_out = L - n_init - n_local - (1 if (pool > 0 and pool % 2 == 0) else 0)
                assert S == n_init + k + n_local, what
                best = torch.sort(votes[b, :n_out], descending=True, stable=True).indices[:k]
                expect = torch.sort(best).values + n_init
                assert torch.equal(sel_pos[b, n_init:n_init + k].long(), expect), what
                assert torch.equal(sel_pos[b, :n_init].cpu(), torch.arange(n_init, dtype=torch.int32))
                assert torch.equal(sel_pos[b, n_init + k:S].cpu(),
                                   torch.arange(L - n_local, L, dtype=torch.int32))
                pos = sel_pos[b, :S].long()
                slots = wl.batch.table[b].long()[pos // page] * page + pos % page
                assert torch.equal(sel[b, :S].long(), slots), what


@pytest.mark.parametrize("fused_select", [True, False], indirect=True, ids=["fused", "separate"])
def test_decode_layer_max_pool(dev, fused_select):
    lens, ks = [5000, 100, 2048, 901], [256, 256, 200, 256]
    say(f"decode_layer with max-pool, fused={fused_select}")
    wl = small(dev, SHAPES[0], seed=71, lens=lens, ks=ks, page=16, top_k=256, n_init=16, n_local=32,
               pool_kernel=9)
    check_layer(wl, dev, "decode_layer max-pool")


def test_topk_ties_and_extremes(dev):
    say("topk ties / k=1 / k=n-1")
    shape = SHAPES[0]
    for n_extra, k in [(50, 1), (50, 49), (3000, 17)]:
        L = 8 + 16 + n_extra
        wl = small(dev, shape, seed=5, lens=[L], ks=[k], top_k=k)
        n = L - 24
        # all-equal votes -> the k lowest positions
        votes = torch.full((1, ops.score_stride_for(L)), 0.25, dtype=torch.float32, device=dev)
        sel, pos, slen = ops.topk_ragged(wl.cfg, wl.batch, votes)
        assert torch.equal(pos[0, 8:8 + k].cpu(), torch.arange(8, 8 + k, dtype=torch.int32))
        # tie-free random votes -> argsort
        g = torch.Generator().manual_seed(n)
        v = torch.rand(n, generator=g)
        votes[0, :n] = v.to(dev)
        sel, pos, slen = ops.topk_ragged(wl.cfg, wl.batch, votes)
        ref = torch.sort(torch.argsort(v, descending=True)[:k]).values + 8
        assert torch.equal(pos[0, 8:8 + k].cpu().long(), ref)
        # negative and mixed-sign values keep their order
        v2 = torch.randn(n, generator=g)
        votes[0, :n] = v2.to(dev)
        sel, pos, slen = ops.topk_ragged(wl.cfg, wl.batch, votes)
        ref = torch.sort(torch.argsort(v2, descending=True)[:k]).values + 8
        assert torch.equal(pos[0, 8:8 + k].cpu().long(), ref)


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"H{s['num_heads']}kv{s['num_kv_heads']}")
@pytest.mark.parametrize("rope_mode", ["ROPE_LLAMA", "NONE"])
def test_sparse_attention(dev, shape, rope_mode):
    say(f"attention H={shape['num_heads']} Hkv={shape['num_kv_heads']} rope={rope_mode}")
    wl = small(dev, shape, seed=11, lens=[2000, 300], ks=[64, 64])
    c = wl.cfg
    c.rope_mode = rope_mode
    g = torch.Generator().manual_seed(3)
    lens = [700, 37]
    sel = torch.zeros((2, 700), dtype=torch.int32)
    for b, S in enumerate(lens):
        sel[b, :S] = torch.randperm(wl.k_pool.shape[0], generator=g)[:S].int()
    sel_len = torch.tensor(lens, dtype=torch.int32)
    out = ops.sparse_decode_attention(c, wl.q, wl.k_pool, wl.v_pool, sel.to(dev), sel_len.to(dev))
    kc, vc, qc = wl.k_pool.cpu(), wl.v_pool.cpu(), wl.q.cpu()
    for b, S in enumerate(lens):
        ref = oracle.attend.sparse_decode_attention(
            qc[b].view(c.num_heads, 128), kc, vc, sel[b, :S], 128 ** -0.5, c.rope_theta, 1.0, 0.0,
            rope_mode)
        err = (out[b].cpu().float() - ref.reshape(-1).float()).abs().max().item()
        assert err <= 2e-2, f"attention b={b}: max abs err {err}"


@pytest.mark.parametrize("B,S", [(1, 40000), (3, 23456)])
def test_attention_over_a_long_dense_list(dev, B, S):
    """A dense request attends over every token (tr.py:377-378, 741-744): lists of tens of
    thousands of entries, 64 workgroups of hundreds of tokens per KV head, a wavefront's
    rotation advanced over dozens of steps; against the oracle in fp32."""
    say(f"attention over dense lists B={B} S={S}")
    wl = small(dev, SHAPES[0], seed=45, lens=[S] * B, ks=[64] * B)
    c = wl.cfg
    g = torch.Generator().manual_seed(46)
    lens = [S - 777 * b for b in range(B)]
    sel = torch.stack([torch.randperm(wl.k_pool.shape[0], generator=g)[:S] for _ in range(B)]).int()
    sel_len = torch.tensor(lens, dtype=torch.int32)
    out = ops.sparse_decode_attention(c, wl.q, wl.k_pool, wl.v_pool, sel.to(dev), sel_len.to(dev))
    torch.cuda.synchronize()
    kc, vc, qc = wl.k_pool.cpu(), wl.v_pool.cpu(), wl.q.cpu()
    for b in range(B):
        ref = oracle.attend.sparse_decode_attention(
            qc[b].view(c.num_heads, 128), kc, vc, sel[b, :lens[b]], 128 ** -0.5, c.rope_theta, 1.0, 0.0, c.rope_mode)
        err = (out[b].cpu().float() - ref.reshape(-1).float()).abs().max().item()
        assert err <= 2e-2, f"b={b}: max abs err {err}"


@pytest.mark.parametrize("B", [1, 14])
def test_attention_never_reads_a_row_it_was_not_given(dev, B):
    """A KV pool as a server holds it: only the rows in use hold numbers.  Every row that no
    list names is filled with NaN, and the entries of `sel` past the lengths point at such rows
    (or outside the pool): a token past a range has the weight zero, but 0 x NaN is NaN, so the
    kernel must not fetch those rows at all.  One request (one tile per wavefront) and 14."""
    lens = [2541] if B == 1 else [2600, 2599, 2541, 1025, 700, 333, 65, 64, 33, 17, 1, 0, 2600, 1800]
    width = 2600
    say(f"attention over a pool with NaN in every unused row B={B}")
    wl = small(dev, SHAPES[0], seed=43, lens=[3000] * B, ks=[64] * B)
    c = wl.cfg
    P = wl.k_pool.shape[0]
    g = torch.Generator().manual_seed(44)
    used = torch.zeros(P, dtype=torch.bool)
    sel = torch.zeros((B, width), dtype=torch.int32)
    for b, S in enumerate(lens):
        rows = torch.randint(0, P - 1, (S,), generator=g)     # (the pool's last row stays unused)
        used[rows] = True
        sel[b, :S] = rows.int()
        sel[b, S:] = torch.where(torch.arange(width - S) % 2 == 0, 0x7fffffff, P - 1).int()
    k_pool, v_pool = wl.k_pool.clone(), wl.v_pool.clone()
    k_pool[~used.to(dev)] = float("nan")
    v_pool[~used.to(dev)] = float("nan")
    sel_len = torch.tensor(lens, dtype=torch.int32)
    out = ops.sparse_decode_attention(c, wl.q, k_pool, v_pool, sel.to(dev), sel_len.to(dev))
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out.float()).all()), "NaN from a row that no list names"
    kc, vc, qc = wl.k_pool.cpu(), wl.v_pool.cpu(), wl.q.cpu()
    for b, S in enumerate(lens):
        if S == 0:
            assert not bool(out[b].any())
            continue
        ref = oracle.attend.sparse_decode_attention(
            qc[b].view(c.num_heads, 128), kc, vc, sel[b, :S], 128 ** -0.5, c.rope_theta, 1.0, 0.0, c.rope_mode)
        assert (out[b].cpu().float() - ref.reshape(-1).float()).abs().max().item() <= 2e-2


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"H{s['num_heads']}kv{s['num_kv_heads']}")
@pytest.mark.parametrize("rope_mode,cap", [("ROPE_LLAMA", 0.0), ("NONE", 0.0), ("ROPE_LLAMA", 25.0)])
def test_sparse_attention_of_many_requests(dev, shape, rope_mode, cap):
    """Many requests with long lists: a workgroup walks several tiles, every head shape, with
    and without the rotation and the soft cap; ragged lengths that end inside a tile, inside a
    wavefront's range, at one entry and at none; the one-request launch of the same lists (one
    tile per wavefront, other ranges) agrees to the rounding of the output."""
    say(f"attention of many requests H={shape['num_heads']} Hkv={shape['num_kv_heads']} {rope_mode} cap={cap}")
    lens = [2600, 2599, 2541, 1025, 700, 333, 65, 64, 33, 17, 1, 0, 2600, 1800]
    B, width = len(lens), 2600
    wl = small(dev, shape, seed=41, lens=[3000] * B, ks=[64] * B)
    c = wl.cfg
    c.rope_mode, c.logit_cap = rope_mode, cap
    g = torch.Generator().manual_seed(42)
    sel = torch.zeros((B, width), dtype=torch.int32)
    for b, S in enumerate(lens):
        sel[b, :S] = torch.randint(0, wl.k_pool.shape[0], (S,), generator=g).int()
        sel[b, S:] = 0x7fffffff     # entries past the length are never used
    sel_len = torch.tensor(lens, dtype=torch.int32)
    out = ops.sparse_decode_attention(c, wl.q, wl.k_pool, wl.v_pool, sel.to(dev), sel_len.to(dev))
    torch.cuda.synchronize()
    kc, vc, qc = wl.k_pool.cpu(), wl.v_pool.cpu(), wl.q.cpu()
    for b, S in enumerate(lens):
        if S == 0:
            assert not bool(out[b].any()), f"b={b}: empty list"
            continue
        ref = oracle.attend.sparse_decode_attention(
            qc[b].view(c.num_heads, 128), kc, vc, sel[b, :S], 128 ** -0.5, c.rope_theta, 1.0, cap, rope_mode)
        err = (out[b].cpu().float() - ref.reshape(-1).float()).abs().max().item()
        assert err <= 2e-2, f"attention b={b} S={S}: max abs err {err}"
        alone = ops.sparse_decode_attention(c, wl.q[b:b + 1], wl.k_pool, wl.v_pool, sel[b:b + 1].to(dev),
                                            sel_len[b:b + 1].to(dev))
        # (the same fp32-equivalent arithmetic over other ranges: a unit of the output's rounding)
        assert (alone[0].float() - out[b].float()).abs().max().item() <= 2 ** -6 * max(1.0, out[b].float().abs().max().item())


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"H{s['num_heads']}kv{s['num_kv_heads']}")
def test_selection_cache_decisions(dev, shape):
    """ts_selcache_step on its own, every head shape (4 to 32 heads: one to four 16-byte
    pieces of the query per thread): queries at chosen cosines to the cached one on both sides
    of the threshold, decisions, cached queries and counters against the oracle's state
    machine over twelve steps."""
    say(f"selection cache decisions H={shape['num_heads']}")
    B = 6
    wl = small(dev, shape, seed=57, lens=[3000] * B, ks=[64] * B)
    c = wl.cfg
    dim = c.num_heads * c.head_dim
    cache = ops.SelectionCache.allocate(c, B, dev)
    refs = [oracle.selcache.SelectionCache() for _ in range(B)]
    g = torch.Generator().manual_seed(58)
    base = torch.randn(B, dim, generator=g)
    for step in range(12):
        # a mix of the anchor direction and a fresh one: cosines from -0.2 to 1.0, several near 0.9
        mix = torch.tensor([1.0, 0.95, 0.9, 0.88, 0.5, -0.2])[torch.randperm(B, generator=g)]
        fresh = torch.randn(B, dim, generator=g)
        fresh -= (fresh * base).sum(1, keepdim=True) / (base * base).sum(1, keepdim=True) * base
        fresh *= base.norm(dim=1, keepdim=True) / fresh.norm(dim=1, keepdim=True)
        qf = (mix[:, None] * base + (1 - mix[:, None] ** 2).clamp_min(0).sqrt() * fresh).bfloat16()
        hit = ops.selcache_step(c, wl.batch, qf.to(dev), cache)
        # (a miss stores the query; the selection that would fill cache_len is stood in for)
        cache.cache_len.copy_(torch.full((B,), 64, dtype=torch.int32))
        torch.cuda.synchronize()
        for b in range(B):
            before = refs[b].q_cached
            cos = None if before is None else oracle.selcache.cosine(before.float(), qf[b].float())
            _, ref_hit = refs[b].step(qf[b], lambda: torch.zeros(1))
            if cos is not None and abs(cos - refs[b].threshold) < 1e-4:
                refs[b].q_cached = cache.q_cache[b].cpu().clone()   # too close to call: follow the device
                refs[b].skip_count = int(cache.counters[b, 0])
            else:
                assert bool(hit[b]) == ref_hit, f"step {step} b={b} cosine {cos}"
                assert torch.equal(cache.q_cache[b].cpu(), refs[b].q_cached), f"step {step} b={b}: cached query"
                assert int(cache.counters[b, 0]) == refs[b].skip_count
            base[b] = cache.q_cache[b].cpu().float()    # the anchor: the query of the last miss
        assert cache.counters[:, 1].tolist() == [step + 1] * B


@pytest.mark.parametrize("seed", range(12))
def test_sparse_attention_randomised(dev, seed):
    """Random batches and ragged list lengths through the decode attention: one pass or
    several per workgroup, one round of workgroups, requests with empty and with one-entry
    lists, any head shape, with or without the rotation and the soft cap; every replay of
    the same call bit-identical (the splits are merged in a fixed order)."""
    rnd = random.Random(6000 + seed)
    shape = SHAPES[rnd.randrange(len(SHAPES))]
    B = rnd.choice([1, 2, rnd.randrange(3, 9), rnd.randrange(9, 25)])
    max_sel = rnd.choice([rnd.randrange(1, 130), rnd.randrange(130, 1500), rnd.randrange(1500, 5000)])
    lens = [rnd.choice([max_sel, rnd.randrange(0, max_sel + 1), rnd.randrange(0, max_sel + 1), 1]) for _ in range(B)]
    lens[rnd.randrange(B)] = max_sel
    rope_mode = rnd.choice(["ROPE_LLAMA", "ROPE_LLAMA", "NONE"])
    cap = rnd.choice([0.0, 0.0, 20.0])
    say(f"attention randomised seed={seed} H={shape['num_heads']} kv={shape['num_kv_heads']} B={B} "
        f"max_sel={max_sel} {rope_mode} cap={cap}")
    wl = small(dev, shape, seed=6100 + seed, lens=[3000] * B, ks=[64] * B)
    c = wl.cfg
    c.rope_mode, c.logit_cap = rope_mode, cap
    g = torch.Generator().manual_seed(6200 + seed)
    sel = torch.zeros((B, max_sel), dtype=torch.int32)
    for b, S in enumerate(lens):
        sel[b, :S] = torch.randint(0, wl.k_pool.shape[0], (S,), generator=g).int()
    sel_len = torch.tensor(lens, dtype=torch.int32)
    out = ops.sparse_decode_attention(c, wl.q, wl.k_pool, wl.v_pool, sel.to(dev), sel_len.to(dev)).clone()
    again = ops.sparse_decode_attention(c, wl.q, wl.k_pool, wl.v_pool, sel.to(dev), sel_len.to(dev))
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), again.view(torch.int16))
    kc, vc, qc = wl.k_pool.cpu(), wl.v_pool.cpu(), wl.q.cpu()
    for b, S in enumerate(lens):
        if S == 0:      # an empty list attends to nothing: the output is defined as zero
            assert not bool(out[b].any()), f"b={b}: empty list"
            continue
        ref = oracle.attend.sparse_decode_attention(
            qc[b].view(c.num_heads, 128), kc, vc, sel[b, :S], 128 ** -0.5, c.rope_theta, 1.0, cap,
            rope_mode)
        err = (out[b].cpu().float() - ref.reshape(-1).float()).abs().max().item()
        assert err <= 2e-2, f"attention b={b} S={S}: max abs err {err}"


def test_attention_soft_cap(dev):
    say("attention logit_cap=30")
    wl = small(dev, SHAPES[0], seed=12, lens=[500], ks=[64])
    c = wl.cfg
    c.logit_cap = 30.0
    c.sm_scale = 1.0  # large logits so the cap bites
    S = 256
    sel = torch.arange(S, dtype=torch.int32).view(1, S)
    out = ops.sparse_decode_attention(c, wl.q, wl.k_pool, wl.v_pool, sel.to(dev),
                                      torch.tensor([S], dtype=torch.int32, device=dev))
    ref = oracle.attend.sparse_decode_attention(wl.q.cpu()[0].view(c.num_heads, 128), wl.k_pool.cpu(),
                                                wl.v_pool.cpu(), sel[0], 1.0, c.rope_theta, 1.0, 30.0)
    assert (out[0].cpu().float() - ref.reshape(-1).float()).abs().max().item() <= 2e-2


@pytest.fixture
def fused_select(request):
    """Runs the layer with the cooperative score + vote kernel (True) or with the
    separate kernels (False); restores the library default afterwards."""
    previous = ops.set_fused_select(request.param)
    yield request.param
    ops.set_fused_select(previous)


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"H{s['num_heads']}kv{s['num_kv_heads']}")
@pytest.mark.parametrize("lens", [[3000], [2500, 700, 3000]], ids=["B1", "B3"])
def test_layer_starts_with_the_selection_on_a_clean_workspace(dev, shape, lens):
    """From its second call of a shape on, a layer object without a selection cache tells the
    library that its workspace is clean (the attention kernel of the call before cleared the
    selection's counters) and the call starts with the selection kernel, which rotates the
    query itself: selections and outputs bit-identical to those of a fresh object, whose first
    call runs the rotation kernel, step after step with new queries; a call of another shape,
    with a selection cache or split at the vote in between makes the next call a full one."""
    say(f"layer on a clean workspace H={shape['num_heads']} kv={shape['num_kv_heads']} B={len(lens)}")
    wl = small(dev, shape, seed=71, lens=lens, ks=[64] * len(lens))
    c, B = wl.cfg, len(lens)
    layer = ops.DecodeLayer(c, B, max(lens), dev)
    layer.workspace.fill_(0xa5)          # whatever an allocation holds
    gen = torch.Generator(device=dev).manual_seed(72)
    cache = ops.SelectionCache.allocate(c, B, dev)
    for step in range(6):
        q = torch.randn(wl.q.shape, device=dev, generator=gen).to(wl.q.dtype)
        was_clean = layer._clean_for
        if step == 3:      # a call with the selection cache: the call after it is a full one
            layer(q, wl.k_pool, wl.v_pool, wl.batch, cache=cache)
            assert layer._clean_for is None
            continue
        if step == 5:      # another shape (one request fewer tokens than the object was sized for)
            import dataclasses
            bt = dataclasses.replace(wl.batch, max_seq_len=max(lens) - 1)
            layer(q, wl.k_pool, wl.v_pool, bt)
            assert layer._clean_for == (B, max(lens) - 1)
            continue
        got = [t.clone() for t in layer(q, wl.k_pool, wl.v_pool, wl.batch)]
        assert layer._clean_for == (B, max(lens))
        assert (was_clean == (B, max(lens))) == (step in (1, 2)), f"step {step}: {was_clean}"
        fresh = ops.DecodeLayer(c, B, max(lens), dev)
        want = fresh(q, wl.k_pool, wl.v_pool, wl.batch)
        torch.cuda.synchronize()
        assert not layer.gave_up() and not fresh.gave_up()
        assert torch.equal(got[3], want[3]), f"step {step}: lengths"
        for b in range(B):
            S = int(want[3][b])
            assert torch.equal(got[1][b, :S], want[1][b, :S]) and torch.equal(got[2][b, :S], want[2][b, :S]), \
                f"step {step} b={b}: selection"
        assert torch.equal(got[0].view(torch.int16), want[0].view(torch.int16)), f"step {step}: output"


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"H{s['num_heads']}kv{s['num_kv_heads']}")
@pytest.mark.parametrize("mode", ["cache", "plain", "paged", "paged-cache"])
@pytest.mark.parametrize("fused_select", [True, False], indirect=True, ids=["fused", "separate"])
def test_decode_step_is_store_then_layer(dev, shape, mode, fused_select):
    """ts_decode_step (the reference's decode forward in one call, tr.py:777-825) against
    ts_kv_store followed by ts_decode_layer over a few steps of AR(1) queries: pools,
    tables, lengths, selections, outputs and the cache's counters bit-identical.  With the
    selection cache and caller-chosen slots the store rides in the layer's first launch;
    with a page pool the slots come from the table and the pool as the paged store takes them
    (2047 and 3000 tokens: one request on a page boundary at the third step, one at the first);
    without the cache the call is the two calls in a row.  A request whose table is full is left
    untouched by both."""
    import dataclasses
    paged = mode.startswith("paged")
    page = 16 if paged else 1
    lens, steps = [3000, 700, 2047], 5
    say(f"decode_step H={shape['num_heads']} kv={shape['num_kv_heads']} mode={mode}")
    wl = small(dev, shape, seed=81, lens=lens, ks=[64] * len(lens), page=page, extra_pages=len(lens) * (steps + 2))
    c, B = wl.cfg, len(lens)
    gen = torch.Generator(device=dev).manual_seed(82)
    qs = workloads.ar1_queries(B, c.num_heads * c.head_dim, steps, dev)
    row = c.num_kv_heads * c.head_dim
    cols = -(-(max(lens) + steps) // page)
    cols = max(cols, wl.table.shape[1])
    results = []
    for fused in (True, False):
        k_pool, v_pool = wl.k_pool.clone(), wl.v_pool.clone()
        table = torch.zeros((B, cols), dtype=torch.int32, device=dev)
        table[:, :wl.table.shape[1]] = wl.table
        if not paged:
            table = table[:, :max(lens) + 3].contiguous()   # the longest request's table fills up at step 3
        seq = wl.seq_lens_dev.clone()
        cache = ops.SelectionCache.allocate(c, B, dev) if mode.endswith("cache") else None
        pages = ops.PagePool.of(wl.free_pages.clone()) if paged else None
        free = wl.free_pages[:B * steps].view(steps, B) if not paged else None
        layer = ops.DecodeLayer(c, B, max(lens) + steps, dev)
        g2 = torch.Generator(device=dev).manual_seed(83)
        trace = []
        for t in range(steps):
            k_new = torch.randn((B, row), generator=g2, device=dev).bfloat16()
            v_new = torch.randn((B, row), generator=g2, device=dev).bfloat16()
            bt = ops.Batch(seq, table, min(max(lens) + t + 1, table.shape[1] * page))
            loc = None if pages else free[t].contiguous()
            if fused:
                got = layer.step(qs[t], k_new, v_new, loc, k_pool, v_pool, bt, cache, pages=pages)
            else:
                ops.kv_store(c, k_new, v_new, loc, k_pool, v_pool, table, seq, pages=pages)
                got = layer(qs[t], k_pool, v_pool, bt, cache)
            torch.cuda.synchronize()
            assert not layer.gave_up()
            trace.append([x.clone() for x in got] + [seq.clone(), table.clone()])
        results.append((trace, k_pool, v_pool, None if cache is None else cache.counters.clone(),
                        None if pages is None else (int(pages.free_count), int(pages.ticket))))
    (ta, ka, va, ca, pa), (tb, kb, vb, cb, pb) = results
    assert pa == pb and (pa is None or pa[1] == 0)
    assert torch.equal(ka, kb) and torch.equal(va, vb)
    if ca is not None:
        assert torch.equal(ca, cb)
    for t, (x, y) in enumerate(zip(ta, tb)):
        assert torch.equal(x[4], y[4]) and torch.equal(x[5], y[5]), f"step {t}: lengths / table"
        assert torch.equal(x[3], y[3]), f"step {t}: selection lengths"
        for b in range(B):
            S = int(x[3][b])
            assert torch.equal(x[1][b, :S], y[1][b, :S]) and torch.equal(x[2][b, :S], y[2][b, :S]), f"step {t} b={b}"
        assert torch.equal(x[0].view(torch.int16), y[0].view(torch.int16)), f"step {t}: output"
    if not paged:   # the first request's table was full from step 3 on: its length stayed
        assert int(ta[-1][4][0]) == max(lens) + 3


def check_layer(wl, dev, tag):
    lens = wl.seq_lens
    layer = ops.DecodeLayer(wl.cfg, len(lens), max(lens), dev)
    out, sel, sel_pos, sel_len = layer(wl.q, wl.k_pool, wl.v_pool, wl.batch)
    torch.cuda.synchronize()
    details = []
    ref_sel, ref_out = oracle_layer(wl, details)
    for b in range(len(lens)):
        S = int(sel_len[b])
        assert S == ref_sel[b].shape[0]
        if details[b]:
            c = wl.cfg
            assert_index_sets_match(sel_pos[b, c.n_init:S - c.n_local].cpu(), details[b]["top_pos"],
                                    details[b]["votes"], c.n_init, f"{tag} top-k b={b}")
        assert_attention_close(wl, b, out[b], sel[b, :S], ref_sel[b], ref_out[b], f"{tag} b={b}")
    return sel_pos, sel_len


@pytest.mark.parametrize("shape", SHAPES[:2], ids=lambda s: f"H{s['num_heads']}kv{s['num_kv_heads']}")
@pytest.mark.parametrize("page", [1, 16])
@pytest.mark.parametrize("fused_select", [True, False], indirect=True, ids=["fused", "separate"])
def test_decode_layer(dev, shape, page, fused_select):
    lens, ks = [5000, 100, 2048, 901], [256, 256, 200, 256]
    say(f"decode_layer H={shape['num_heads']} page={page} lens={lens} fused={fused_select}")
    wl = small(dev, shape, seed=21 + page, lens=lens, ks=ks, page=page, top_k=256, n_init=16,
               n_local=32)
    check_layer(wl, dev, "decode_layer")


@pytest.mark.parametrize("seed", range(12))
def test_decode_layer_randomised(dev, seed):
    """Random batches through ts_decode_layer against the oracle, whatever form the layer
    takes for them (one selection launch, the phased votes-only launch + top-k kernels, the
    separate kernels): 1 to 14 requests of 40 to 40 000 tokens, ragged k, any head shape,
    pages of 1 or 16, lengths on the host too or not, with or without max-pooling."""
    rnd = random.Random(9000 + seed)
    shape = SHAPES[rnd.randrange(len(SHAPES))]
    B = rnd.randrange(1, 15)
    lens = [rnd.choice([rnd.randrange(40, 400), rnd.randrange(400, 6000), rnd.randrange(6000, 40000)])
            for _ in range(B)]
    top_k = rnd.choice([16, 64, 256])
    ks = [rnd.randrange(1, top_k + 1) for _ in range(B)]
    pool_kernel = rnd.choice([-1, -1, 5, 8])
    fused = rnd.random() < 0.8
    wl = small(dev, shape, seed=9100 + seed, lens=lens, ks=ks, page=rnd.choice([1, 16]), top_k=top_k,
               n_init=rnd.choice([4, 16]), n_local=rnd.choice([8, 32]), pool_kernel=pool_kernel)
    wl.host_lengths = rnd.random() < 0.5
    previous = ops.set_fused_select(fused)
    try:
        form = ops.layer_selection_form(wl.cfg, wl.batch)
        say(f"decode_layer randomised seed={seed} H={shape['num_heads']} kv={shape['num_kv_heads']} B={B} "
            f"tokens={sum(lens)} pool={pool_kernel} host_lengths={wl.host_lengths} form={form}")
        check_layer(wl, dev, f"randomised layer seed={seed}")
    finally:
        ops.set_fused_select(previous)


@pytest.mark.parametrize("fused_select", [True, False], indirect=True, ids=["fused", "separate"])
def test_decode_layer_object_serves_smaller_batches(dev, fused_select):
    """A layer object sized for the largest batch and context is called with batches of
    changing size and length, as a serving loop does; every call gives what a fresh
    object of exactly that size gives."""
    say(f"decode_layer: one object, changing batches, fused={fused_select}")
    shape = SHAPES[0]
    big = None
    for seed, lens, ks in ((31, [5000, 100, 2048, 901], [256, 256, 200, 256]),
                           (32, [700], [256]),
                           (33, [6000, 3000, 5999, 64, 1200], [256, 100, 256, 256, 7]),
                           (34, [2500, 2600], [256, 256])):
        wl = small(dev, shape, seed=seed, lens=lens, ks=ks, page=16, top_k=256, n_init=16, n_local=32)
        big = big or ops.DecodeLayer(wl.cfg, 5, 6000, dev)
        out, sel, sel_pos, sel_len = [t.clone() for t in big(wl.q, wl.k_pool, wl.v_pool, wl.batch)]
        fresh = ops.DecodeLayer(wl.cfg, len(lens), max(lens), dev)
        out2, sel2, pos2, len2 = fresh(wl.q, wl.k_pool, wl.v_pool, wl.batch)
        torch.cuda.synchronize()
        assert torch.equal(sel_len, len2), f"lens={lens}"
        for b in range(len(lens)):
            S = int(sel_len[b])
            assert torch.equal(sel_pos[b, :S], pos2[b, :S]) and torch.equal(sel[b, :S], sel2[b, :S])
        assert torch.equal(out.view(torch.int16), out2.view(torch.int16)), f"lens={lens}"


@pytest.mark.parametrize("shape", SHAPES[2:], ids=lambda s: f"H{s['num_heads']}kv{s['num_kv_heads']}")
@pytest.mark.parametrize("fused_select", [True], indirect=True, ids=["fused"])
def test_decode_layer_fused_shapes(dev, shape, fused_select):
    lens, ks = [3001, 40, 1500], [128, 128, 100]
    say(f"decode_layer fused H={shape['num_heads']}kv{shape['num_kv_heads']} lens={lens}")
    wl = small(dev, shape, seed=77, lens=lens, ks=ks, page=16, top_k=128)
    check_layer(wl, dev, "decode_layer fused")


@pytest.mark.parametrize("fused_select", [True, False], indirect=True, ids=["fused", "separate"])
def test_decode_layer_many_chunks(dev, fused_select):
    """Long ragged batch: hundreds of workgroups per request meet at the grid-wide
    rendezvous and the statistics merge walks more than 64 chunks per head."""
    lens, ks = [70000, 9000, 33000], [1024, 512, 1024]
    say(f"decode_layer long lens={lens} fused={fused_select}")
    wl = small(dev, SHAPES[0], seed=5, lens=lens, ks=ks, page=16, top_k=1024, n_init=128,
               n_local=512)
    check_layer(wl, dev, "decode_layer long")


@pytest.mark.parametrize("fused_select", [True], indirect=True, ids=["fused"])
def test_decode_layer_fused_full_lds(dev, fused_select):
    """Four 64K requests: the largest batch whose scores still fit the LDS of the
    device (512 candidates per workgroup, more than 64 KB of LDS each)."""
    lens, ks = [65536, 65536, 60000, 65536], [2048, 2048, 2048, 1000]
    say(f"decode_layer fused, LDS-filling batch lens={lens}")
    wl = small(dev, SHAPES[0], seed=9, lens=lens, ks=ks, page=1, top_k=2048, n_init=128,
               n_local=512)
    assert ops.select_supported(wl.cfg, len(lens), max(lens))
    check_layer(wl, dev, "decode_layer full LDS")


def test_max_pool_votes(dev):
    for kernel in (5, 6, 32):
        say(f"max-pool kernel={kernel}")
        wl = small(dev, SHAPES[0], seed=31, lens=[2500, 900], ks=[64, 64], pool_kernel=kernel)
        c = wl.cfg
        qf = fingerprint(wl, dev)
        scores, partials = ops.score(c, wl.batch, qf, wl.k_pool)
        votes, stats = ops.vote(c, wl.batch, scores, partials)
        sel, sel_pos, sel_len = ops.topk_ragged(c, wl.batch, votes)
        details = []
        oracle_layer(wl, details)
        for b, L in enumerate(wl.seq_lens):
            n_out = details[b]["votes"].shape[0]
            assert torch.allclose(votes[b, :n_out].cpu(), details[b]["votes"], rtol=2e-4, atol=1e-9)
            S = int(sel_len[b])
            assert_index_sets_match(sel_pos[b, c.n_init:S - c.n_local].cpu(), details[b]["top_pos"],
                                    details[b]["votes"], c.n_init, f"pooled top-k b={b}", rtol=3e-4)


def test_kv_store(dev):
    say("kv_store")
    wl = small(dev, SHAPES[0], seed=41, lens=[100, 50], ks=[16, 16], extra_pages=8)
    c = wl.cfg
    table = torch.zeros((2, 128), dtype=torch.int32, device=dev)
    table[:, :wl.table.shape[1]] = wl.table
    seq = wl.seq_lens_dev.clone()
    loc = torch.tensor([wl.k_pool.shape[0] - 1, wl.k_pool.shape[0] - 2], dtype=torch.int32, device=dev)
    k = torch.randn(2, c.num_kv_heads * 128, device=dev).bfloat16()
    v = torch.randn(2, c.num_kv_heads * 128, device=dev).bfloat16()
    ops.kv_store(c, k, v, loc, wl.k_pool, wl.v_pool, table, seq)
    assert seq.tolist() == [101, 51]
    assert table[0, 100].item() == loc[0].item() and table[1, 50].item() == loc[1].item()
    assert torch.equal(wl.k_pool[loc[0].item()].reshape(-1), k[0])
    assert torch.equal(wl.v_pool[loc[1].item()].reshape(-1), v[1])


@pytest.mark.parametrize("pool_kernel", [-1, 6])
def test_score_vote_in_groups_of_requests(dev, pool_kernel):
    """ts_score_vote (scores never in memory, the batch served in phases of requests)
    against the oracle's votes and against ts_score + ts_vote; ragged, with a dense
    request and a skipped one."""
    lens, ks = [3000, 777, 40, 1531, 2048, 900], [64] * 6
    say(f"score_vote lens={lens} pool={pool_kernel}")
    wl = small(dev, SHAPES[0], seed=41, lens=lens, ks=ks, page=16, top_k=64, pool_kernel=pool_kernel)
    c = wl.cfg
    assert ops.score_vote_supported(c, len(lens), max(lens))
    qf = fingerprint(wl, dev)
    skip = torch.tensor([0, 0, 0, 1, 0, 0], dtype=torch.int32, device=dev)
    details = []
    oracle_layer(wl, details)
    votes_sep, _ = ops.vote(c, wl.batch, *ops.score(c, wl.batch, qf, wl.k_pool, skip=skip), skip=skip)
    votes = ops.score_vote(c, wl.batch, qf, wl.k_pool, skip=skip)
    # the same with the lengths (here: upper bounds of them) known on the host: the launches are
    # then packed by what the requests hold, and workgroups without candidates stay out
    bounds = torch.tensor([min(L + 100, max(lens)) for L in lens], dtype=torch.int32)
    packed = ops.Batch(wl.batch.seq_lens, wl.batch.table, max(lens), wl.batch.k_per_req,
                       host_seq_lens=bounds)
    votes_packed = ops.score_vote(c, packed, qf, wl.k_pool, skip=skip)
    torch.cuda.synchronize()
    for b, L in enumerate(lens):
        if not details[b] or b == 3:
            continue
        n = L - c.n_init - c.n_local
        if pool_kernel > 0 and pool_kernel % 2 == 0:
            n -= 1
        ref = details[b]["votes"][:n]
        for name, v in (("grouped", votes), ("packed", votes_packed)):
            got = v[b, :n].cpu()
            assert (got - ref).abs().max().item() <= 2e-4 * ref.abs().max().item(), f"{name} b={b}"
            assert (got - votes_sep[b, :n].cpu()).abs().max().item() <= 1e-5 * ref.abs().max().item()


@pytest.mark.parametrize("case", ["many small requests", "a dozen long requests"])
@pytest.mark.parametrize("pool_kernel", [-1, 5])
def test_score_vote_phases_of_one_launch(dev, case, pool_kernel):
    """With the lengths on the host the votes-only form packs the requests into phases and
    puts the workgroups of many phases into one grid, which the device works through in
    order: 200 small requests make more phases than one launch holds (eight requests to a
    phase), a dozen long ones make phases of a few requests that take turns on the device.
    Against ts_score + ts_vote on the same inputs; the host's lengths are upper bounds, two
    requests are dense, some are skipped."""
    rnd = random.Random(5)
    if case == "many small requests":
        lens = [rnd.randrange(700, 3000) for _ in range(200)]
        lens[17], lens[150] = 40, 80
    else:
        lens = [rnd.randrange(20000, 60000) for _ in range(12)]
        lens[5] = 300
    B = len(lens)
    say(f"score_vote in phases: {case}, pool={pool_kernel}")
    wl = small(dev, SHAPES[0], seed=47, lens=lens, ks=[64] * B, page=16, top_k=64, pool_kernel=pool_kernel)
    c = wl.cfg
    qf = fingerprint(wl, dev)
    skip = torch.tensor([1 if b % 11 == 3 else 0 for b in range(B)], dtype=torch.int32, device=dev)
    votes_sep, _ = ops.vote(c, wl.batch, *ops.score(c, wl.batch, qf, wl.k_pool, skip=skip), skip=skip)
    bounds = torch.tensor([min(L + rnd.randrange(0, 700), max(lens)) for L in lens], dtype=torch.int32)
    packed = ops.Batch(wl.batch.seq_lens, wl.batch.table, max(lens), wl.batch.k_per_req,
                       host_seq_lens=bounds)
    for attempt in range(2):  # (the second call finds the workspace as the first one left it)
        votes = ops.score_vote(c, packed, qf, wl.k_pool, skip=skip)
        torch.cuda.synchronize()
        for b, L in enumerate(lens):
            n = L - c.n_init - c.n_local
            if pool_kernel > 0 and pool_kernel % 2 == 0:
                n -= 1
            if L <= c.n_init + 64 + c.n_local or skip[b]:   # dense: no votes are taken
                continue
            want = votes_sep[b, :n]
            assert (votes[b, :n] - want).abs().max().item() <= 1e-5 * want.abs().max().item(), \
                f"b={b} L={L} attempt={attempt}"


@pytest.mark.parametrize("shape", SHAPES[1:], ids=lambda s: f"H{s['num_heads']}kv{s['num_kv_heads']}")
def test_score_vote_phases_head_shapes(dev, shape):
    """The phased votes-only launch for the other head shapes (seven and eight query heads per
    KV head run one workgroup per CU, one KV head streams 256-byte rows): 40 requests, five
    phases, against ts_score + ts_vote."""
    rnd = random.Random(9)
    lens = [rnd.randrange(700, 6000) for _ in range(40)]
    say(f"score_vote in phases: H={shape['num_heads']} kv={shape['num_kv_heads']}")
    wl = small(dev, shape, seed=49, lens=lens, ks=[64] * 40, page=16, top_k=64)
    c = wl.cfg
    qf = fingerprint(wl, dev)
    votes_sep, _ = ops.vote(c, wl.batch, *ops.score(c, wl.batch, qf, wl.k_pool))
    for host in (None, torch.tensor(lens, dtype=torch.int32)):
        bt = ops.Batch(wl.batch.seq_lens, wl.batch.table, max(lens), wl.batch.k_per_req, host_seq_lens=host)
        votes = ops.score_vote(c, bt, qf, wl.k_pool)
        torch.cuda.synchronize()
        for b, L in enumerate(lens):
            n = L - c.n_init - c.n_local
            want = votes_sep[b, :n]
            assert (votes[b, :n] - want).abs().max().item() <= 1e-5 * want.abs().max().item(), \
                f"b={b} L={L} host lengths: {host is not None}"


@pytest.mark.parametrize("seed", range(16))
def test_score_vote_randomised(dev, seed):
    """Random batches through the phased votes-only launch against ts_score + ts_vote: 1 to 40
    requests of 30 to 30 000 tokens (some dense), random slack in the host's bounds or no
    bounds at all, random skip flags, with or without max-pooling, one of the head shapes."""
    rnd = random.Random(7000 + seed)
    shape = SHAPES[rnd.randrange(len(SHAPES))]
    B = rnd.randrange(1, 41)
    lens = [rnd.choice([rnd.randrange(30, 300), rnd.randrange(300, 4000), rnd.randrange(4000, 30000)])
            for _ in range(B)]
    pool_kernel = rnd.choice([-1, -1, 3, 6])
    say(f"score_vote randomised seed={seed} H={shape['num_heads']} kv={shape['num_kv_heads']} B={B} "
        f"pool={pool_kernel}")
    wl = small(dev, shape, seed=7100 + seed, lens=lens, ks=[32] * B, page=rnd.choice([1, 16]), top_k=32,
               pool_kernel=pool_kernel)
    c = wl.cfg
    qf = fingerprint(wl, dev)
    skip = torch.tensor([1 if rnd.random() < 0.15 else 0 for _ in range(B)], dtype=torch.int32, device=dev)
    host = None
    if rnd.random() < 0.7:
        host = torch.tensor([min(L + rnd.choice([0, 0, 5, 900]), max(lens)) for L in lens], dtype=torch.int32)
    bt = ops.Batch(wl.batch.seq_lens, wl.batch.table, max(lens), wl.batch.k_per_req, host_seq_lens=host)
    votes_sep, _ = ops.vote(c, wl.batch, *ops.score(c, wl.batch, qf, wl.k_pool, skip=skip), skip=skip)
    votes = ops.score_vote(c, bt, qf, wl.k_pool, skip=skip)
    torch.cuda.synchronize()
    for b, L in enumerate(lens):
        n = L - c.n_init - c.n_local
        if pool_kernel > 0 and pool_kernel % 2 == 0:
            n -= 1
        if L <= c.n_init + 32 + c.n_local or skip[b] or n <= 0:   # dense or skipped: no votes are taken
            continue
        want = votes_sep[b, :n]
        assert (votes[b, :n] - want).abs().max().item() <= 1e-5 * want.abs().max().item(), f"b={b} L={L}"


def test_score_vote_reports_a_length_above_its_bound(dev):
    """host_seq_lens are upper bounds; a request that is longer on the device than the host
    said has no workgroups for its last tokens.  The launch says so at once (the caller's
    fault word, without waiting for statistics that cannot come), and the same call with
    honest bounds on the same workspace is correct."""
    import time
    lens = [3000, 2000, 2500]
    say(f"score_vote with a bound below the length, lens={lens}")
    wl = small(dev, SHAPES[0], seed=53, lens=lens, ks=[64] * 3, page=16, top_k=64)
    c = wl.cfg
    qf = fingerprint(wl, dev)
    word = ops.fault_word()
    space = ops.select_workspace(c, wl.batch, dev)
    low = ops.Batch(wl.batch.seq_lens, wl.batch.table, max(lens), wl.batch.k_per_req, word,
                    host_seq_lens=torch.tensor([1400, 2000, 2500], dtype=torch.int32))
    torch.cuda.synchronize()
    t0 = time.time()
    ops.score_vote(c, low, qf, wl.k_pool, workspace=space)
    torch.cuda.synchronize()
    assert time.time() - t0 < 1.0, "reported without running into the bound of a wait"
    with pytest.raises(ops.SelectionGaveUp):
        ops.raise_if_gave_up(word)
    word.zero_()
    good = ops.Batch(wl.batch.seq_lens, wl.batch.table, max(lens), wl.batch.k_per_req, word,
                     host_seq_lens=torch.tensor(lens, dtype=torch.int32))
    votes = ops.score_vote(c, good, qf, wl.k_pool, workspace=space)
    votes_sep, _ = ops.vote(c, wl.batch, *ops.score(c, wl.batch, qf, wl.k_pool))
    torch.cuda.synchronize()
    ops.raise_if_gave_up(word)
    for b, L in enumerate(lens):
        n = L - c.n_init - c.n_local
        want = votes_sep[b, :n]
        assert (votes[b, :n] - want).abs().max().item() <= 1e-5 * want.abs().max().item(), f"b={b}"


@pytest.mark.parametrize("pool_kernel", [-1, 5])
@pytest.mark.parametrize("fused_select", [True, False], indirect=True, ids=["fused", "separate"])
def test_layer_split_at_the_vote(dev, fused_select, pool_kernel):
    """ts_decode_layer_votes + ts_decode_layer_attend give what ts_decode_layer gives; and two
    ranks that hold half of the heads each select, from the sum of their votes, what one
    rank with all heads selects (tr.py:361-364), each attending with its own heads."""
    lens, ks = [2500, 100, 1800], [128, 128, 100]
    say(f"layer split at the vote, fused={fused_select} pool={pool_kernel}")
    wl = small(dev, SHAPES[0], seed=43, lens=lens, ks=ks, page=16, top_k=128, n_init=16, n_local=32,
               pool_kernel=pool_kernel)
    c, B = wl.cfg, 3
    c.head_map = "div"      # a rank holds whole GQA groups: heads [r*H/2, (r+1)*H/2) and their KV heads
    whole = ops.DecodeLayer(c, B, max(lens), dev)
    out, sel, sel_pos, sel_len = [t.clone() for t in whole(wl.q, wl.k_pool, wl.v_pool, wl.batch)]
    halves = ops.DecodeLayer(c, B, max(lens), dev)
    votes = halves.votes(wl.q, wl.k_pool, wl.batch)
    out2, sel2, pos2, len2 = halves.attend(wl.q, votes, wl.k_pool, wl.v_pool, wl.batch)
    torch.cuda.synchronize()
    assert torch.equal(sel_len, len2)
    for b in range(B):
        S = int(sel_len[b])
        assert torch.equal(sel[b, :S], sel2[b, :S]) and torch.equal(sel_pos[b, :S], pos2[b, :S])
    assert (out.float() - out2.float()).abs().max().item() <= 1e-3
    # two ranks
    H, Hkv, D = c.num_heads, c.num_kv_heads, c.head_dim
    import copy
    rc = copy.copy(c)
    rc.num_heads, rc.num_kv_heads = H // 2, Hkv // 2
    ranks = []
    for r in range(2):
        q_r = wl.q.view(B, H, D)[:, r * H // 2:(r + 1) * H // 2].contiguous().view(B, -1)
        k_r = wl.k_pool[:, r * Hkv // 2:(r + 1) * Hkv // 2].contiguous()
        v_r = wl.v_pool[:, r * Hkv // 2:(r + 1) * Hkv // 2].contiguous()
        layer = ops.DecodeLayer(rc, B, max(lens), dev)
        ranks.append((layer, q_r, k_r, v_r, layer.votes(q_r, k_r, wl.batch).clone()))
    total = ranks[0][4] + ranks[1][4]               # the all-reduce
    details = []
    oracle_layer(wl, details) if False else None
    for r, (layer, q_r, k_r, v_r, _) in enumerate(ranks):
        out_r, sel_r, pos_r, len_r = layer.attend(q_r, total, k_r, v_r, wl.batch)
        torch.cuda.synchronize()
        assert torch.equal(len_r, sel_len)
        for b in range(B):
            S = int(sel_len[b])
            same = torch.equal(pos_r[b, :S], sel_pos[b, :S])
            if not same:   # the sum over heads in another order may move a tie at the k-th vote
                n = lens[b] - c.n_init - c.n_local
                v = total[b, :n].cpu()
                assert_index_sets_match(pos_r[b, c.n_init:S - c.n_local].cpu(),
                                        sel_pos[b, c.n_init:S - c.n_local].cpu().long(), v, c.n_init,
                                        f"rank {r} b={b}") if pool_kernel <= 0 else None
            else:
                want = out.view(B, H, D)[b, r * H // 2:(r + 1) * H // 2].reshape(-1).float()
                assert (out_r[b].float() - want).abs().max().item() <= 2e-2


def test_selection_form_agrees_with_what_the_launchers_serve(dev):
    """ts_decode_layer picks its selection form from the very plans its launchers follow: over
    a sweep of head shapes, batches, lengths and pooling windows the form is 2 exactly where
    ts_select serves, 1 exactly where only ts_score_vote does, and a per-call switch to the
    separate kernels gives 0 without touching the process-wide setting."""
    import dataclasses
    say("selection form sweep")
    seen = set()
    for shape in SHAPES:
        for pool_kernel in (-1, 5, 300):
            for B in (1, 2, 4, 16, 64):
                for L in (700, 5000, 65536, 131072, 262144, 1048000):
                    c = ops.LayerConfig(page_size=16, n_init=128, n_local=512, top_k=2048,
                                        pool_kernel=pool_kernel, **shape)
                    form = ops.layer_selection_form(c, B, L)
                    sel_ok = ops.select_supported(c, B, L)
                    vote_ok = ops.score_vote_supported(c, B, L)
                    want = 2 if sel_ok else (1 if vote_ok else 0)
                    assert form == want, (shape, pool_kernel, B, L, form, sel_ok, vote_ok)
                    seen.add(form)
    assert seen == {0, 1, 2}
    wl = small(dev, SHAPES[0], seed=5, lens=[3000], ks=[64])
    assert ops.layer_selection_form(wl.cfg, wl.batch) == 2
    assert ops.layer_selection_form(wl.cfg, dataclasses.replace(wl.batch, separate_kernels=True)) == 0
    assert ops.layer_selection_form(wl.cfg, wl.batch) == 2


@pytest.mark.parametrize("shape", [SHAPES[0], SHAPES[1], SHAPES[6]],
                         ids=lambda s: f"H{s['num_heads']}kv{s['num_kv_heads']}")
def test_fused_select_with_a_threshold_hint(dev, shape):
    """ts_batch.threshold_hint: the selection notes the bin of the k-th vote and, given it
    back, publishes what its last round needs before the first rendezvous, so that one
    rendezvous is enough.  The result is that of a launch without a hint, bit for bit: with
    the right hint (one round met for), with hints off by a few bins inside the band, with
    hints outside it and with nonsense (two rounds again), and for another query whose
    threshold has moved."""
    import dataclasses
    L, k = 40000, 512
    say(f"fused select with a threshold hint H={shape['num_heads']} L={L}")
    wl = small(dev, shape, seed=101, lens=[L], ks=[k], page=16, top_k=k, n_init=128, n_local=512)
    c = wl.cfg
    qf = fingerprint(wl, dev)
    space = ops.select_workspace(c, wl.batch, dev)
    want = ops.select(c, wl.batch, qf, wl.k_pool, workspace=space)[:3]
    torch.cuda.synchronize()
    assert ops.select_rounds(c, wl.batch, space)[:2][1] > 0, "without a hint: a second round"
    hint = torch.zeros(1, dtype=torch.int32, device=dev)
    hinted = dataclasses.replace(wl.batch, hint=hint)

    def run(q=qf, expect=want):
        got = ops.select(c, hinted, q, wl.k_pool, workspace=space)[:3]
        torch.cuda.synchronize()
        assert not ops.select_fault(c, hinted, space)
        for name, x, y in zip(("sel", "sel_pos", "sel_len"), got, expect):
            assert torch.equal(x, y), name
        return ops.select_rounds(c, hinted, space)

    assert run()[1] > 0                 # no hint yet: the usual two rounds, and the hint is left
    code = int(hint[0])
    assert 1 <= code <= 2048
    assert run()[1] == 0                # the right hint: one round
    for off in (-3, -1, 1, 4):          # the band [hint - 4, hint + 3] still holds the bin
        hint.fill_(code + off)
        assert run()[1] == 0, off
        assert int(hint[0]) == code
    for off in (-4, 5, 300, -code):     # it does not, or there is no hint at all: the list round is back
        hint.fill_(code + off)
        assert run()[1] > 0, off
        assert int(hint[0]) == code
    hint.fill_(5000)                    # nonsense
    assert run()[1] > 0
    # another query: its own selection, whatever the old hint says
    g = torch.Generator(device=dev).manual_seed(102)
    q2 = (qf.float() + 0.3 * torch.randn(qf.shape, generator=g, device=dev)).bfloat16()
    want2 = ops.select(c, wl.batch, q2, wl.k_pool, workspace=space)[:3]
    run(q2, want2)
    run(q2, want2)


def test_fused_select_hint_with_ties_and_a_batch(dev):
    """The band path where it is hardest: exact ties at the k-th vote inside and across
    workgroups (duplicated key rows), and a batch whose requests differ in length, one of them
    dense; the second launch (hints set by the first) equals the first."""
    import dataclasses
    lens, ks = [9000, 40, 5200, 7000], [256, 64, 100, 256]
    say(f"fused select with hints, ties, lens={lens}")
    wl = small(dev, SHAPES[0], seed=103, lens=lens, ks=ks, page=16, top_k=256)
    c = wl.cfg
    # duplicate rows: every candidate of request 0 shares its key row with two others
    tabs = cpu_tabs(wl)
    rows = tabs[0][c.n_init:lens[0] - c.n_local].long().to(dev)
    src = rows[torch.arange(rows.shape[0], device=dev) // 3 * 3]
    wl.k_pool[rows] = wl.k_pool[src]
    qf = fingerprint(wl, dev)
    space = ops.select_workspace(c, wl.batch, dev)
    want = ops.select(c, wl.batch, qf, wl.k_pool, workspace=space)[:3]
    hint = torch.zeros(len(lens), dtype=torch.int32, device=dev)
    hinted = dataclasses.replace(wl.batch, hint=hint)
    for launch in range(3):
        got = ops.select(c, hinted, qf, wl.k_pool, workspace=space)[:3]
        torch.cuda.synchronize()
        assert not ops.select_fault(c, hinted, space)
        assert torch.equal(got[2], want[2])
        for b in range(len(lens)):
            S = int(want[2][b])
            assert torch.equal(got[0][b, :S], want[0][b, :S]), (launch, b)
            assert torch.equal(got[1][b, :S], want[1][b, :S]), (launch, b)
    assert int(hint[1]) == 0 and all(int(hint[b]) > 0 for b in (0, 2, 3))
    # and against the oracle
    votes = ops.select(c, wl.batch, qf, wl.k_pool, want_votes=True, workspace=space)[3]
    torch.cuda.synchronize()
    for b in (0, 2, 3):
        n = lens[b] - c.n_init - c.n_local
        v = votes[b, :n].cpu()
        order = sorted(range(n), key=lambda t: (-v[t].item(), t))[:ks[b]]
        S = int(got[2][b])
        assert sorted(order) == (got[1][b, c.n_init:S - c.n_local] - c.n_init).tolist(), b
