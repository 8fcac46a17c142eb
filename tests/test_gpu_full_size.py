"""The benchmark configurations at their full sizes: the whole layer against the
CPU oracle where the oracle finishes in seconds (one or two requests at a time),
and properties that do not depend on the size (every head's softmax sums to one,
the selection is the exact top-k of the votes, ascending positions between the
sink and the local window, slots = table[positions], bit-stable reruns, planted
critical tokens are selected far above chance, the selection cache's counters add
up)."""

import pytest
import torch

import oracle
from tokenselect_amd import ops, workloads
from helpers import assert_attention_close, assert_index_sets_match, say

pytestmark = pytest.mark.gpu


def _sm(c):
    return c.sm_scale if c.sm_scale is not None else c.head_dim ** -0.5


def _oracle_requests(wl, requests, details):
    c = wl.cfg
    table = wl.table.cpu()
    tabs = [oracle.select.expand_page_table(table[b], wl.seq_lens[b], c.page_size) for b in requests]
    H, D = c.num_heads, c.head_dim
    return oracle.layer.decode_layer(
        wl.q.view(len(wl.seq_lens), H * D)[requests].cpu(), wl.k_pool.cpu(), wl.v_pool.cpu(), tabs,
        [wl.seq_lens[b] for b in requests], H, D, c.n_init, c.n_local,
        [wl.k_list[b] for b in requests], c.rope_theta, c.rope_scale, _sm(c), details=details)


def _votes_on_device(wl):
    """The library's own votes [B, stride], from the path the layer takes for this shape
    (the two paths may differ in the last bit of a vote), and the rotated query."""
    c, bt, B = wl.cfg, wl.batch, len(wl.seq_lens)
    cos, sin = ops.scoring_cos_sin(c.head_dim, c.rope_theta, c.rope_scale, c.n_local, wl.q.device)
    qf = ops.rope_apply(wl.q.view(B, c.num_heads, c.head_dim), cos, sin, None)
    form = ops.layer_selection_form(c, bt)
    if form == 2:
        return ops.select(c, bt, qf, wl.k_pool, want_votes=True)[3], qf
    if form == 1:
        return ops.score_vote(c, bt, qf, wl.k_pool), qf
    scores, partials = ops.score(c, bt, qf, wl.k_pool)
    return ops.vote(c, bt, scores, partials)[0], qf


def _check_properties(wl, layer_out, votes, tag):
    c = wl.cfg
    out, sel, sel_pos, sel_len = layer_out
    for b, (L, k) in enumerate(zip(wl.seq_lens, wl.k_list)):
        S = int(sel_len[b])
        pos = sel_pos[b, :S].long()
        tab = oracle.select.expand_page_table(wl.table[b].cpu(), L, c.page_size).to(pos.device)
        assert torch.equal(sel[b, :S].long(), tab[pos].long()), f"{tag} b={b}: slots != table[pos]"
        if c.n_init + k + c.n_local >= L:
            assert S == L and torch.equal(pos, torch.arange(L, device=pos.device))
            continue
        n = L - c.n_init - c.n_local
        assert S == c.n_init + k + c.n_local
        assert torch.equal(pos[:c.n_init], torch.arange(c.n_init, device=pos.device))
        assert torch.equal(pos[-c.n_local:], torch.arange(L - c.n_local, L, device=pos.device))
        mid = pos[c.n_init:S - c.n_local]
        assert bool((mid[1:] > mid[:-1]).all()), f"{tag} b={b}: positions not ascending"
        assert int(mid[0]) >= c.n_init and int(mid[-1]) < L - c.n_local
        v = votes[b, :n]
        total = v.double().sum().item()       # every head's probabilities sum to one
        assert abs(total - c.num_heads) <= 1e-3 * c.num_heads, (tag, b, total)
        chosen = torch.zeros(n, dtype=torch.bool, device=v.device)
        chosen[mid - c.n_init] = True
        assert int(chosen.sum()) == k
        # exact top-k: nothing left out beats anything taken; ties go to the lower position
        lowest_in, highest_out = v[chosen].min(), v[~chosen].max()
        assert float(lowest_in) >= float(highest_out), (tag, b)
        tied_in = torch.nonzero(chosen & (v == lowest_in)).flatten()
        tied_out = torch.nonzero(~chosen & (v == lowest_in)).flatten()
        if tied_out.numel():
            assert int(tied_in.max()) < int(tied_out.min()), f"{tag} b={b}: tie order"


def _check_against_oracle(wl, layer_out, requests, tag):
    c = wl.cfg
    out, sel, sel_pos, sel_len = layer_out
    details = []
    ref_sel, ref_out = _oracle_requests(wl, requests, details)
    for i, b in enumerate(requests):
        S = int(sel_len[b])
        assert S == ref_sel[i].shape[0]
        if details[i]:
            assert_index_sets_match(sel_pos[b, c.n_init:S - c.n_local].cpu(), details[i]["top_pos"],
                                    details[i]["votes"], c.n_init, f"{tag} b={b}")
        assert_attention_close(wl, b, out[b], sel[b, :S], ref_sel[i], ref_out[i], f"{tag} b={b}")


def _run(wl, dev):
    layer = ops.DecodeLayer(wl.cfg, len(wl.seq_lens), max(wl.seq_lens), dev)
    first = [t.clone() for t in layer(wl.q, wl.k_pool, wl.v_pool, wl.batch)]
    again = layer(wl.q, wl.k_pool, wl.v_pool, wl.batch)
    torch.cuda.synchronize()
    for x, y in zip(first, again):        # bit-stable: no result depends on atomics' order
        assert torch.equal(x, y)
    return first


@pytest.mark.parametrize("fused", [True, False], ids=["fused", "separate"])
@pytest.mark.parametrize("config", ["config1", "config2"])
def test_single_request_configs(dev, config, fused):
    previous = ops.set_fused_select(fused)
    try:
        wl = getattr(workloads, config)(dev)
        say(f"full size {wl.name} fused={fused}")
        result = _run(wl, dev)
        votes, _ = _votes_on_device(wl)
        _check_properties(wl, result, votes, wl.name)
        _check_against_oracle(wl, result, [0], wl.name)
        if wl.planted:      # the tokens shifted along the query direction are the critical ones
            S = int(result[3][0])
            mid = set(result[2][0, wl.cfg.n_init:S - wl.cfg.n_local].tolist())
            planted = set(wl.planted[0].tolist())
            recall = len(mid & planted) / len(planted)
            chance = wl.cfg.top_k / (wl.seq_lens[0] - wl.cfg.n_init - wl.cfg.n_local)
            say(f"  planted tokens selected: {recall:.3f} (chance {chance:.3f})")
            assert recall >= 20 * chance     # about half of them in practice
    finally:
        ops.set_fused_select(previous)


def test_scores_at_full_size_against_a_dense_product(dev):
    """ts_score at the 128K configuration against fp32 torch products on the device for
    4096 sampled candidates of every head (1e-3 of the score scale)."""
    wl = workloads.config2(dev)
    say(f"full size scores {wl.name}")
    c, bt = wl.cfg, wl.batch
    L = wl.seq_lens[0]
    _, qf = _votes_on_device(wl)
    scores = ops.scores_head_major(c, ops.score(c, bt, qf, wl.k_pool)[0])   # [B, H, stride]
    g = torch.Generator(device=dev).manual_seed(1)
    t = torch.randperm(L - c.n_init - c.n_local, generator=g, device=dev)[:4096]
    tab = oracle.select.expand_page_table(wl.table[0].cpu(), L, c.page_size).to(dev)
    rows = wl.k_pool[tab[t + c.n_init].long()].float()                       # [4096, Hkv, D]
    q = qf.view(c.num_heads, c.head_dim).float()
    kv_of = torch.arange(c.num_heads, device=dev) % c.num_kv_heads          # tr.py:202
    ref = torch.einsum("hd,thd->ht", q, rows[:, kv_of])
    got = scores[0, :, t]
    scale = ref.pow(2).mean().sqrt().item()
    assert (got - ref).abs().max().item() <= 1e-3 * scale


@pytest.mark.parametrize("host_lengths,fused", [(False, True), (True, True), (False, False)],
                         ids=["device-lengths", "host-lengths", "separate-kernels"])
def test_ragged_batch_config(dev, host_lengths, fused):
    """The batch is too large for one co-resident launch: it is scored and voted on as phases
    of one launch (form 1), packed by the host's lengths where the batch carries them and by
    max_seq_len where not; with the fused kernels switched off, by the separate kernels."""
    previous = ops.set_fused_select(fused)
    try:
        wl = workloads.config3(dev)
        wl.host_lengths = host_lengths
        say(f"full size {wl.name} lens={wl.seq_lens} host_lengths={host_lengths} fused={fused}")
        assert ops.layer_selection_form(wl.cfg, wl.batch) == (1 if fused else 0)
        result = _run(wl, dev)
        votes, _ = _votes_on_device(wl)
        _check_properties(wl, result, votes, wl.name)
        order = sorted(range(len(wl.seq_lens)), key=lambda b: wl.seq_lens[b])
        _check_against_oracle(wl, result, [order[0], order[len(order) // 2], order[-1]], wl.name)
    finally:
        ops.set_fused_select(previous)


def test_large_context_layer_config(dev):
    wl = workloads.config5_layer(dev)
    say(f"full size {wl.name}")
    result = _run(wl, dev)
    votes, _ = _votes_on_device(wl)
    _check_properties(wl, result, votes, wl.name)
    _check_against_oracle(wl, result, [3], wl.name)


def test_selection_cache_trace_config(dev):
    """The 64-step trace: hits + misses = lookups, a hit reuses the positions of the last
    miss, a miss selects afresh (checked against the oracle on the last miss)."""
    steps = 64
    wl = workloads.config4(dev, steps=steps)
    say(f"full size {wl.name}")
    c, B, L0 = wl.cfg, len(wl.seq_lens), wl.seq_lens[0]
    qs = workloads.ar1_queries(B, c.num_heads * c.head_dim, steps, dev)
    g = torch.Generator(device=dev).manual_seed(7)
    k_new = torch.randn((steps, B, c.num_kv_heads * c.head_dim), generator=g, device=dev).bfloat16()
    v_new = torch.randn((steps, B, c.num_kv_heads * c.head_dim), generator=g, device=dev).bfloat16()
    free = torch.arange(B * L0, B * (L0 + steps), dtype=torch.int32, device=dev).view(steps, B)
    table = torch.zeros((B, L0 + steps), dtype=torch.int32, device=dev)
    table[:, :L0] = wl.table[:, :L0]
    seq = wl.seq_lens_dev.clone()
    cache = ops.SelectionCache.allocate(c, B, dev)
    layer = ops.DecodeLayer(c, B, L0 + steps, dev)
    previous_mid, hits_seen, last_miss = None, 0, None
    cos_t, sin_t = ops.scoring_cos_sin(c.head_dim, c.rope_theta, c.rope_scale, c.n_local, dev)
    anchors = [None] * B          # the oracle's state machine: fingerprint of the last miss
    for t in range(steps):
        before = cache.counters.clone()
        ops.kv_store(c, k_new[t], v_new[t], free[t], wl.k_pool, wl.v_pool, table, seq)
        out, sel, sel_pos, sel_len = layer(qs[t], wl.k_pool, wl.v_pool, ops.Batch(seq, table, L0 + t + 1),
                                           cache)
        torch.cuda.synchronize()
        L = L0 + t + 1
        S = c.n_init + c.top_k + c.n_local
        assert sel_len.tolist() == [S] * B
        mid = sel_pos[:, c.n_init:S - c.n_local].clone()
        assert torch.equal(sel_pos[:, S - c.n_local:S].cpu(),
                           torch.arange(L - c.n_local, L, dtype=torch.int32).repeat(B, 1))
        hit = (cache.counters[:, 0] - before[:, 0]).tolist()
        assert (cache.counters[:, 1] - before[:, 1]).tolist() == [1] * B
        # every step's decision against the oracle's cosine rule on the same fingerprints
        qf = ops.rope_apply(qs[t].view(B, c.num_heads, c.head_dim), cos_t, sin_t, None).cpu()
        for b in range(B):
            fp = qf[b].reshape(-1)
            if anchors[b] is None:
                assert not hit[b], f"step {t} b={b}: the first lookup must miss"
            else:
                cos = oracle.selcache.cosine(anchors[b], fp)
                want = cos >= oracle.selcache.THRESHOLD
                if want != bool(hit[b]):            # only a cosine on the threshold may differ
                    assert abs(cos - oracle.selcache.THRESHOLD) < 1e-5, (t, b, cos, hit[b])
            if not hit[b]:
                anchors[b] = fp.clone()
        for b in range(B):
            if hit[b]:
                hits_seen += 1
                assert torch.equal(mid[b], previous_mid[b]), f"step {t} b={b}: a hit must reuse"
            else:
                last_miss = (t, b, qs[t, b].clone(), mid[b].clone(), L)
        previous_mid = mid
    assert 0 < hits_seen < steps * B
    assert int(cache.counters[:, 0].sum()) == hits_seen
    # the last miss of the trace against the oracle (the pool only grew since then)
    t, b, q, mid, L = last_miss
    d = {}
    oracle.select.retrieval_indices(q.view(1, -1).cpu(), wl.k_pool.cpu(), table[b].cpu(), L, c.num_heads,
                                    c.head_dim, c.n_init, c.n_local, c.top_k, c.rope_theta,
                                    c.rope_scale, detail=d)
    assert_index_sets_match(mid.cpu(), d["top_pos"], d["votes"], c.n_init, f"trace step {t} b={b}")
