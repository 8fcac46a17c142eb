"""Pins the CPU oracle.  The reference has no tests, golden vectors or fixtures
for this path, and its module cannot be imported here (SGLang / vLLM /
FlashInfer / CUDA), so every oracle function is checked against something the
mathematics fixes: an independent formulation, a library routine, a closed
form, an invariant, or brute force on tiny inputs.  None of the checks retypes
the oracle's own expression."""

import math

import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import attend, rope, selcache, select


def rnd(*shape, seed=0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype)


# ------------------------------------------------------------------- RoPE
def complex_rope(x, pos, base, scale=1.0):
    """Independent formulation: pair (i, i+D/2) is a complex number multiplied by
    exp(i * pos * scale * base^(-2i/D)), evaluated in float64."""
    d = x.shape[-1]
    half = d // 2
    xc = torch.complex(x[..., :half].double(), x[..., half:].double())
    freq = torch.tensor([base ** (-2.0 * i / d) for i in range(half)], dtype=torch.float64)
    ang = pos.double().view(-1, 1, 1) * scale * freq
    rot = xc * torch.polar(torch.ones_like(ang), ang)
    return torch.cat((rot.real, rot.imag), dim=-1)


@pytest.mark.parametrize("base", [1e4, 5e5, 1e6])
def test_rope_matches_complex_multiplication(base):
    x = rnd(7, 3, 128, seed=1, dtype=torch.float32)
    pos = torch.tensor([0, 1, 2, 17, 512, 513, 4000])
    got = rope.apply(x, pos, base)
    ref = complex_rope(x, pos, base)
    # fp32 tables: angle error ~ pos * 2^-24, so compare at 1e-3 absolute for pos <= 4000
    assert (got.double() - ref).abs().max() < 2e-3
    assert (got[:5].double() - ref[:5]).abs().max() < 2e-4


def test_rope_position_zero_is_identity_and_norm_is_kept():
    x = rnd(4, 2, 128, seed=2)
    assert torch.equal(rope.apply(x, torch.zeros(4, dtype=torch.long), 5e5), x)
    xf = x.float()
    y = rope.apply(xf, torch.tensor([5, 77, 512, 1023]), 5e5)
    pair_norm = lambda t: t[..., :64] ** 2 + t[..., 64:] ** 2
    assert torch.allclose(pair_norm(y), pair_norm(xf), rtol=1e-5, atol=1e-5)


def test_rope_relative_position_property():
    q, k = rnd(1, 4, 128, seed=3, dtype=torch.float32), rnd(1, 4, 128, seed=4, dtype=torch.float32)
    for a, b in [(512, 100), (30, 29), (700, 0)]:
        lhs = (rope.apply(q, torch.tensor([a]), 1e4) * rope.apply(k, torch.tensor([b]), 1e4)).sum(-1)
        rhs = (rope.apply(q, torch.tensor([a - b]), 1e4) * k).sum(-1)
        assert torch.allclose(lhs, rhs, rtol=1e-4, atol=1e-3)


def test_rope_distance_scale_multiplies_the_position():
    x = rnd(1, 2, 128, seed=5, dtype=torch.float32)
    assert torch.allclose(rope.apply(x, torch.tensor([6]), 1e4, distance_scale=2),
                          rope.apply(x, torch.tensor([12]), 1e4), atol=1e-5)


def test_scoring_query_rotates_to_n_local_and_rounds_to_bf16():
    q = rnd(1, 4 * 128, seed=6)
    qf = rope.scoring_query(q, 4, 128, 512, 5e5)
    assert qf.dtype == torch.bfloat16 and qf.shape == (512,)
    ref = complex_rope(q.view(1, 4, 128).float(), torch.tensor([512]), 5e5).view(-1)
    assert (qf.double() - ref).abs().max() < 0.02  # one bf16 rounding of values ~N(0,1)
    # two rows: positions n_local and n_local+1, then the mean over rows
    q2 = rnd(2, 4 * 128, seed=7)
    qf2 = rope.scoring_query(q2, 4, 128, 16, 1e4)
    ref2 = complex_rope(q2.view(2, 4, 128).float(), torch.tensor([16, 17]), 1e4).view(2, -1).mean(0)
    assert (qf2.double() - ref2).abs().max() < 0.03


# ------------------------------------------------------------------ score
def brute_score(qf, k_pool, cand, mapping):
    H, D = qf.shape
    out = torch.zeros(H, len(cand), dtype=torch.float64)
    for h in range(H):
        for t, slot in enumerate(cand.tolist()):
            acc = 0.0
            for d in range(D):
                acc += float(qf[h, d]) * float(k_pool[slot, mapping(h), d])
            out[h, t] = acc
    return out


def test_score_brute_force_and_head_map_discriminator():
    H, Hkv, D, P = 4, 2, 16, 12
    qf, k_pool = rnd(H, D, seed=8), rnd(P, Hkv, D, seed=9)
    cand = torch.tensor([5, 0, 11, 3, 7], dtype=torch.int32)
    got = select.score(qf, k_pool, cand)
    mod = brute_score(qf, k_pool, cand, lambda h: h % Hkv)
    div = brute_score(qf, k_pool, cand, lambda h: h // (H // Hkv))
    assert (got.double() - mod).abs().max() < 1e-5           # the reference's h % Hkv
    assert (got.double() - div).abs().max() > 0.5            # and NOT the conventional h // G
    assert (select.score(qf, k_pool, cand, head_map="div").double() - div).abs().max() < 1e-5


def test_score_one_hot_known_answers_and_no_scaling():
    H, Hkv, D, P = 4, 2, 128, 6
    k_pool = torch.zeros(P, Hkv, D, dtype=torch.bfloat16)
    k_pool[3, 1, 10] = 2.0
    k_pool[4, 0, 127] = -3.0
    qf = torch.zeros(H, D, dtype=torch.bfloat16)
    qf[1, 10] = 1.5      # head 1 -> kv head 1
    qf[2, 127] = 4.0     # head 2 -> kv head 0
    s = select.score(qf, k_pool, torch.arange(P, dtype=torch.int32))
    expect = torch.zeros(H, P)
    expect[1, 3] = 3.0   # raw dot product: no 1/sqrt(D)
    expect[2, 4] = -12.0
    expect[3, 3] = 0.0
    assert torch.equal(s, expect)


def test_score_follows_the_table_not_the_pool_order():
    qf, k_pool = rnd(8, 128, seed=10), rnd(64, 2, 128, seed=11)
    perm = torch.randperm(64, generator=torch.Generator().manual_seed(1))
    cand = torch.arange(40, dtype=torch.int32)
    base = select.score(qf, k_pool, cand)
    shuffled_pool = torch.empty_like(k_pool)
    shuffled_pool[perm] = k_pool                      # row r moves to slot perm[r]
    assert torch.equal(select.score(qf, shuffled_pool, perm[:40].int()), base)


# ------------------------------------------------------------- vote / pool
def test_vote_mass_shift_invariance_and_single_head():
    s = rnd(6, 300, seed=14, dtype=torch.float32) * 5
    c = select.vote(s)
    assert abs(c.sum().item() - 6.0) < 1e-4                   # each head contributes mass 1
    shifted = s + torch.tensor([3.0, -7.0, 0.0, 100.0, -50.0, 1.0]).view(6, 1)
    assert torch.allclose(select.vote(shifted), c, rtol=1e-4, atol=1e-7)
    one = s[:1]
    e = torch.exp(one[0].double() - one[0].double().max())
    assert torch.allclose(select.vote(one).double(), e / e.sum(), rtol=1e-5, atol=1e-9)


@pytest.mark.parametrize("kernel", [1, 2, 5, 6, 32])
def test_max_pool_matches_naive_window(kernel):
    v = torch.rand(97, generator=torch.Generator().manual_seed(kernel))
    got = select.max_pool(v, kernel)
    pad = (kernel - 1) // 2
    n_out = 97 + 2 * pad - kernel + 1
    assert got.shape[0] == n_out == (97 if kernel % 2 else 96)   # even kernels lose one element
    for t in (0, 1, n_out // 2, n_out - 1):
        lo, hi = max(t - pad, 0), min(t - pad + kernel, 97)
        assert got[t].item() == v[lo:hi].max().item()
    assert select.max_pool(v, -1) is v and select.max_pool(v, 0) is v


# ------------------------------------------------------------------- top-k
def test_topk_sorted_against_argsort_and_extremes():
    v = torch.rand(500, generator=torch.Generator().manual_seed(15))
    for k in (1, 7, 499):
        ref = sorted(sorted(range(500), key=lambda i: -v[i].item())[:k])
        got = select.topk_sorted(v, k)
        assert got.tolist() == ref
        assert got.dtype == torch.int64
    planted = torch.zeros(100)
    planted[[3, 50, 99]] = torch.tensor([5.0, 7.0, 6.0])
    assert select.topk_sorted(planted, 3).tolist() == [3, 50, 99]


# ---------------------------------------------------------------- assembly
def test_assemble_structure_and_dense_rule():
    L, n_init, n_local, k = 100, 4, 8, 5
    tab = (torch.arange(L, dtype=torch.int32) * 3 + 1)
    top = torch.tensor([10, 20, 21, 50, 91])
    out = select.assemble(tab, L, n_init, n_local, top)
    assert out.shape[0] == n_init + k + n_local and out.dtype == torch.int32
    assert out[:n_init].tolist() == [1, 4, 7, 10]
    assert out[-n_local:].tolist() == [(L - n_local + i) * 3 + 1 for i in range(n_local)]
    assert out[n_init:n_init + k].tolist() == [t * 3 + 1 for t in top.tolist()]
    ident = torch.arange(L, dtype=torch.int32)
    assert select.assemble(ident, L, n_init, n_local, top)[n_init:n_init + k].tolist() == top.tolist()
    assert select.is_dense(17, 4, 8, 5) and not select.is_dense(18, 4, 8, 5)


def test_retrieval_indices_end_to_end_small():
    H, Hkv, D, P, L = 4, 2, 128, 300, 200
    n_init, n_local, k = 4, 8, 16
    k_pool = rnd(P, Hkv, D, seed=16)
    q = rnd(1, H * D, seed=17)
    tab = torch.randperm(P, generator=torch.Generator().manual_seed(2))[:L].int()
    assert select.retrieval_indices(q, k_pool, tab, n_init + k + n_local, H, D, n_init, n_local, k,
                                    1e4) is None
    d = {}
    out = select.retrieval_indices(q, k_pool, tab, L, H, D, n_init, n_local, k, 1e4, detail=d)
    assert out.shape[0] == n_init + k + n_local
    assert out[:n_init].tolist() == tab[:n_init].tolist()
    assert out[-n_local:].tolist() == tab[L - n_local:L].tolist()
    top = d["top_pos"]
    assert top.min() >= n_init and top.max() < L - n_local
    assert bool((top[1:] > top[:-1]).all())
    # independent recomputation: float64 softmax votes over the candidate rows
    qf = complex_rope(q.view(1, H, D).float(), torch.tensor([n_local]), 1e4)[0].to(torch.bfloat16)
    cand = tab[n_init:L - n_local].long()
    s = torch.stack([k_pool[cand, h % Hkv].double() @ qf[h].double() for h in range(H)])
    votes = torch.softmax(s, -1).sum(0)
    ref = torch.sort(torch.topk(votes, k).indices).values + n_init
    assert top.tolist() == ref.tolist()


def test_planted_tokens_dominate_the_selection():
    """Known answer: candidates shifted far along every query's direction must all be selected."""
    H, Hkv, D, P, L = 8, 2, 128, 600, 600
    n_init, n_local, k = 8, 16, 32
    g = torch.Generator().manual_seed(18)
    k_pool = torch.randn(P, Hkv, D, generator=g).bfloat16()
    q = torch.randn(1, H * D, generator=g).bfloat16()
    tab = torch.arange(L, dtype=torch.int32)
    qf = rope.scoring_query(q, H, D, n_local, 1e4).view(H, D).float()
    planted = torch.randperm(L - n_init - n_local, generator=g)[:k] + n_init
    for kvh in range(Hkv):
        direction = qf[kvh::Hkv].mean(0)
        k_pool[planted, kvh] = (k_pool[planted, kvh].float()
                                + 12.0 * direction / direction.norm()).bfloat16()
    d = {}
    select.retrieval_indices(q, k_pool, tab, L, H, D, n_init, n_local, k, 1e4, detail=d)
    assert sorted(d["top_pos"].tolist()) == sorted(planted.tolist())


def test_expand_page_table():
    pt = torch.tensor([7, 2, 9], dtype=torch.int32)
    assert select.expand_page_table(pt, 10, 4).tolist() == [28, 29, 30, 31, 8, 9, 10, 11, 36, 37]
    assert select.expand_page_table(pt, 3, 1).tolist() == [7, 2, 9]


# --------------------------------------------------------------- attention
def sdpa_reference(q, k_pool, v_pool, slots, scale):
    H, Hkv = q.shape[0], k_pool.shape[1]
    k = k_pool[slots.long()].float().permute(1, 0, 2).repeat_interleave(H // Hkv, dim=0)
    v = v_pool[slots.long()].float().permute(1, 0, 2).repeat_interleave(H // Hkv, dim=0)
    return F.scaled_dot_product_attention(q.float().unsqueeze(1), k, v, scale=scale).squeeze(1)


def test_attention_without_rope_is_textbook_sdpa_with_standard_gqa():
    H, Hkv, D, P = 8, 2, 128, 90
    q, k_pool, v_pool = rnd(H, D, seed=19), rnd(P, Hkv, D, seed=20), rnd(P, Hkv, D, seed=21)
    slots = torch.randperm(P, generator=torch.Generator().manual_seed(3))[:40].int()
    got = attend.sparse_decode_attention(q, k_pool, v_pool, slots, D ** -0.5, 1e4, rope_mode="NONE")
    ref = sdpa_reference(q, k_pool, v_pool, slots, D ** -0.5)
    assert got.dtype == torch.bfloat16
    assert (got.float() - ref).abs().max() < 1e-2
    full = attend.sparse_decode_attention(q, k_pool, v_pool, torch.arange(P, dtype=torch.int32),
                                          D ** -0.5, 1e4, rope_mode="NONE")
    assert (full.float() - sdpa_reference(q, k_pool, v_pool, torch.arange(P), D ** -0.5)).abs().max() < 1e-2


def test_attention_rope_positions_are_list_indices():
    """Rotating q to S-1 and key j to j equals SDPA on tensors rotated by the
    independent complex formulation; a common position offset changes nothing."""
    H, Hkv, D, P, S = 4, 2, 128, 70, 33
    q, k_pool, v_pool = rnd(H, D, seed=22), rnd(P, Hkv, D, seed=23), rnd(P, Hkv, D, seed=24)
    slots = torch.randperm(P, generator=torch.Generator().manual_seed(4))[:S].int()
    got = attend.sparse_decode_attention(q, k_pool, v_pool, slots, D ** -0.5, 5e5, rope_scale=1.0)
    for offset in (0, 1000):
        qr = complex_rope(q.float().unsqueeze(0), torch.tensor([S - 1 + offset]), 5e5)[0]
        kr = complex_rope(k_pool[slots.long()].float(), torch.arange(S) + offset, 5e5)
        logits = torch.einsum("hd,shd->hs", qr, kr[:, torch.arange(H) // (H // Hkv)]) * D ** -0.5
        ref = torch.einsum("hs,shd->hd", torch.softmax(logits, -1),
                           v_pool[slots.long()].double()[:, torch.arange(H) // (H // Hkv)])
        assert (got.double() - ref).abs().max() < 1e-2
    scaled = attend.sparse_decode_attention(q, k_pool, v_pool, slots, D ** -0.5, 5e5, rope_scale=4.0)
    assert (scaled.float() - got.float()).abs().max() > 1e-3   # rope_scale divides the angle


def test_attention_soft_cap():
    H, Hkv, D, P = 4, 2, 128, 40
    q, k_pool, v_pool = rnd(H, D, seed=25), rnd(P, Hkv, D, seed=26), rnd(P, Hkv, D, seed=27)
    slots = torch.arange(P, dtype=torch.int32)
    plain = attend.sparse_decode_attention(q, k_pool, v_pool, slots, 1.0, 1e4, rope_mode="NONE")
    huge = attend.sparse_decode_attention(q, k_pool, v_pool, slots, 1.0, 1e4, 1.0, 1e6, "NONE")
    assert (plain.float() - huge.float()).abs().max() < 2e-2   # cap >> logits: no effect
    tight = attend.sparse_decode_attention(q, k_pool, v_pool, slots, 1.0, 1e4, 1.0, 1.0, "NONE")
    k = k_pool.float()[:, torch.arange(H) // 2]
    logits = torch.tanh(torch.einsum("hd,shd->hs", q.float(), k))
    ref = torch.einsum("hs,shd->hd", torch.softmax(logits, -1), v_pool.float()[:, torch.arange(H) // 2])
    assert (tight.float() - ref).abs().max() < 1e-2


# --------------------------------------------------------- selection cache
def test_selection_cache_state_machine():
    assert selcache.THRESHOLD == 0.8984375
    q = rnd(512, seed=28)
    calls = []
    sel = lambda: (calls.append(1), torch.tensor([len(calls)]))[1]
    c = selcache.SelectionCache()
    top, hit = c.step(q, sel)
    assert not hit and top.tolist() == [1]                     # first query always selects
    top, hit = c.step(q, sel)
    assert hit and top.tolist() == [1] and c.skip_count == 1   # cos(q, q) = 1
    top, hit = c.step(-q, sel)
    assert not hit and top.tolist() == [2]                     # cos = -1
    ortho = rnd(512, seed=29)
    ortho = (ortho.float() - (ortho.float() @ (-q).float()) / (q.float() @ q.float()) * (-q).float())
    top, hit = c.step(ortho.bfloat16(), sel)
    assert not hit                                             # cos ~ 0
    assert c.retrieval_count == 4 and c.skip_count == 1


def test_anchor_is_the_last_miss_not_the_previous_query():
    """AR(1) drift: cos to the anchor decays 0.95, 0.9025, 0.857 ... so the
    reference's last-miss anchor re-selects at the third step, while a
    previous-query anchor would keep hitting."""
    g = torch.Generator().manual_seed(30)
    dim, rho = 4096, 0.95
    qs = [torch.randn(dim, generator=g)]
    for _ in range(12):
        qs.append(rho * qs[-1] + math.sqrt(1 - rho * rho) * torch.randn(dim, generator=g))
    ref, alt = selcache.SelectionCache(), selcache.SelectionCache(anchor="previous")
    sel = lambda: torch.tensor([0])
    hits_ref = [ref.step(q.bfloat16(), sel)[1] for q in qs]
    hits_alt = [alt.step(q.bfloat16(), sel)[1] for q in qs]
    assert hits_ref[:4] == [False, True, True, False]
    assert all(hits_alt[1:])
    assert ref.skip_count < alt.skip_count


def test_batched_layer_applies_single_request_semantics():
    H, Hkv, D, P = 4, 2, 128, 400
    k_pool, v_pool = rnd(P, Hkv, D, seed=31), rnd(P, Hkv, D, seed=32)
    q = rnd(2, H * D, seed=33)
    tabs = [torch.arange(0, 250, dtype=torch.int32), torch.arange(250, 278, dtype=torch.int32)]
    sels, out = oracle.layer.decode_layer(q, k_pool, v_pool, tabs, [250, 28], H, D, 4, 8, [16, 16],
                                          1e4, 1.0, D ** -0.5)
    assert sels[0].shape[0] == 28 and sels[1].tolist() == tabs[1].tolist()   # second one is dense
    alone = oracle.layer.decode_layer(q[1:], k_pool, v_pool, tabs[1:], [28], H, D, 4, 8, [16],
                                      1e4, 1.0, D ** -0.5)[1]
    assert torch.equal(out[1], alone[0])


# ---------------------------------------------------------------- chunked prefill
def _prefill_case(seed=0, m=24, S=90, H=4, Hkv=2, P=200):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(m, H, 128, generator=g).bfloat16()
    kp = torch.randn(P, Hkv, 128, generator=g).bfloat16()
    vp = torch.randn(P, Hkv, 128, generator=g).bfloat16()
    slots = torch.randperm(P, generator=g)[:S].int()
    return q, kp, vp, slots


def test_prefill_attention_matches_sdpa_with_explicit_mask():
    """RoPE off: the chunk attention is textbook attention under the mask
    key j visible to row i iff j <= S - m + i."""
    q, kp, vp, slots = _prefill_case()
    m, H, _ = q.shape
    S, G = slots.shape[0], H // kp.shape[1]
    got = oracle.prefill.sparse_prefill_attention(q, kp, vp, slots, 0.11, 1e4, rope_mode="NONE")
    k = kp[slots.long()].float().repeat_interleave(G, dim=1).permute(1, 0, 2)   # [H, S, D]
    v = vp[slots.long()].float().repeat_interleave(G, dim=1).permute(1, 0, 2)
    mask = torch.tril(torch.ones(m, S, dtype=torch.bool), diagonal=S - m)
    ref = torch.nn.functional.scaled_dot_product_attention(
        q.float().permute(1, 0, 2), k, v, attn_mask=mask, scale=0.11).permute(1, 0, 2)
    assert (got.float() - ref).abs().max().item() <= 1e-2


def test_prefill_rows_are_decode_steps_over_key_prefixes():
    """With RoPE on, row i of a chunk equals the decode attention (query at the last
    position) over the first S - m + i + 1 selected keys: pins the query position,
    the key positions and the causal cut at once against the decode oracle."""
    q, kp, vp, slots = _prefill_case(seed=1)
    m, S = q.shape[0], slots.shape[0]
    got = oracle.prefill.sparse_prefill_attention(q, kp, vp, slots, 0.09, 5e5)
    for i in (0, 7, m - 1):
        ref = oracle.attend.sparse_decode_attention(q[i], kp, vp, slots[:S - m + i + 1], 0.09, 5e5)
        assert (got[i].float() - ref.float()).abs().max().item() <= 1e-2
    # not causal: every row sees all keys, so the last row is unchanged and the first is not
    full = oracle.prefill.sparse_prefill_attention(q, kp, vp, slots, 0.09, 5e5, causal=False)
    assert torch.equal(full[m - 1], got[m - 1])
    assert (full[0].float() - got[0].float()).abs().max().item() > 1e-3


def test_prefill_with_fewer_keys_than_rows():
    """S < m (a chunk longer than the selected list, as with the reference's own defaults):
    the first m - S rows sit at negative positions and see no key, so their output is zero;
    every later row is still the decode attention over its key prefix."""
    q, kp, vp, slots = _prefill_case(seed=2, m=40, S=25)
    m, S = q.shape[0], slots.shape[0]
    got = oracle.prefill.sparse_prefill_attention(q, kp, vp, slots, 0.09, 5e5)
    assert torch.count_nonzero(got[:m - S]) == 0
    assert not torch.isnan(got.float()).any()
    for i in (m - S, m - S + 3, m - 1):
        ref = oracle.attend.sparse_decode_attention(q[i], kp, vp, slots[:S - m + i + 1], 0.09, 5e5)
        assert (got[i].float() - ref.float()).abs().max().item() <= 1e-2


def test_prefill_one_row_chunk_is_the_decode_layer():
    g = torch.Generator().manual_seed(5)
    H, Hkv, L = 4, 2, 300
    kp = torch.randn(L, Hkv, 128, generator=g).bfloat16()
    vp = torch.randn(L, Hkv, 128, generator=g).bfloat16()
    q = torch.randn(1, H * 128, generator=g).bfloat16()
    tab = torch.randperm(L, generator=g).int()
    slots, out = oracle.prefill.prefill_chunk(q, kp, vp, tab, L, H, 128, 4, 16, 32, 1e4, 1.0, 0.1)
    ref_slots, ref_out = oracle.layer.decode_layer(q, kp, vp, [tab], [L], H, 128, 4, 16, [32], 1e4,
                                                   1.0, 0.1)
    assert torch.equal(slots, ref_slots[0])
    assert torch.equal(out, ref_out)


def test_prefill_fingerprint_is_the_mean_of_rows_rotated_to_consecutive_positions():
    g = torch.Generator().manual_seed(6)
    rows, H = 40, 2
    q = torch.randn(rows, H * 128, generator=g).bfloat16()
    qf = oracle.rope.scoring_query(q, H, 128, 16, 1e4)
    x = q.view(rows, H, 128).double()
    inv = 1.0 / (1e4 ** (torch.arange(0, 128, 2, dtype=torch.float64) / 128))
    ang = torch.arange(16, 16 + rows, dtype=torch.float64)[:, None] * inv           # [rows, 64]
    z = torch.complex(x[..., :64], x[..., 64:]) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    rot = torch.cat((z.real, z.imag), dim=-1).bfloat16().double()                    # rounded per row
    ref = rot.mean(dim=0).reshape(-1)
    assert (qf.double() - ref).abs().max().item() <= 2.0 ** -8 * ref.abs().max().item()


def test_prefill_loop_stores_then_selects_chunk_by_chunk():
    """The extend loop appends each chunk before selecting for it; a later chunk
    sees the earlier ones among its candidates and every chunk ends with itself."""
    g = torch.Generator().manual_seed(8)
    H, Hkv, L0, T, chunk = 4, 2, 200, 70, 32
    P = L0 + T
    kp = torch.randn(P, Hkv, 128, generator=g).bfloat16()
    vp = torch.randn(P, Hkv, 128, generator=g).bfloat16()
    tab = torch.zeros(P, dtype=torch.int32)
    tab[:L0] = torch.randperm(L0, generator=g).int()
    new_slots = (L0 + torch.randperm(T, generator=g)).int()
    q = torch.randn(T, H * 128, generator=g).bfloat16()
    k_new = torch.randn(T, Hkv, 128, generator=g).bfloat16()
    v_new = torch.randn(T, Hkv, 128, generator=g).bfloat16()
    details = []
    out = oracle.prefill.prefill(q, k_new, v_new, kp, vp, tab, L0, new_slots, H, 128, 4, chunk, 16,
                                 1e4, 1.0, 0.1, chunk=chunk, details=details)
    assert out.shape == (T, H * 128) and len(details) == 3
    assert torch.equal(tab[L0:], new_slots) and torch.equal(kp[new_slots.long()], k_new)
    # chunk 2 (rows 32..63) alone, from the final pools and its own context length
    L2 = L0 + 64
    _, ref = oracle.prefill.prefill_chunk(q[32:64], kp, vp, tab, L2, H, 128, 4, chunk, 16, 1e4, 1.0,
                                          0.1)
    assert torch.equal(out[32:64], ref)


# ------------------------------------------------------------- store / paged append
def test_append_slots_is_the_reference_slice_assignment():
    tab = torch.zeros(10, dtype=torch.int32)
    L = oracle.store.append_slots(tab, 3, torch.tensor([7, 8, 9]), 10)
    assert L == 6 and tab.tolist() == [0, 0, 0, 7, 8, 9, 0, 0, 0, 0]
    assert oracle.store.append_slots(tab, 8, torch.tensor([1, 2, 3]), 10) == 10   # tail dropped
    assert tab[8:].tolist() == [1, 2]


def test_paged_append_matches_what_the_page_arithmetic_fixes():
    ps, pages_cap = 4, 12
    g = torch.Generator().manual_seed(5)
    free = torch.randperm(40, generator=g).tolist()
    table = torch.full((3, pages_cap), -1, dtype=torch.int32)
    lens = [0, 0, 0]
    given = {b: [] for b in range(3)}
    start = len(free)
    for step in range(19):
        slots = oracle.store.append_token_paged(table, lens, free, ps, pages_cap * ps, 40 * ps)
        for b, s in enumerate(slots):
            given[b].append(s)
    assert lens == [19, 19, 19]
    for b in range(3):     # slots are exactly the expanded page table
        assert oracle.select.expand_page_table(table[b], 19, ps).tolist() == given[b]
    used = table[table >= 0].tolist()
    assert len(set(used)) == len(used) == 3 * 5            # ceil(19 / 4) pages each, all distinct
    assert start - len(free) == 15 and not set(used) & set(free)
    # request order, top of the stack first
    free2 = [10, 11, 12]
    t2 = torch.full((2, 4), -1, dtype=torch.int32)
    assert oracle.store.append_token_paged(t2, [0, 4], free2, 4, 16, 1000) == [12 * 4, 11 * 4]
    assert free2 == [10] and t2[0, 0] == 12 and t2[1, 1] == 11
    # page size 1: one slot popped per token
    t3 = torch.full((1, 8), -1, dtype=torch.int32)
    free3 = [5, 6, 7]
    assert oracle.store.append_token_paged(t3, [2], free3, 1, 8, 100) == [7] and free3 == [5, 6]


def test_paged_chunk_equals_token_by_token_and_drops_what_does_not_fit():
    ps = 16
    for L0, rows in ((0, 80), (37, 45), (48, 3), (15, 1), (16, 33)):
        free_a, free_b = list(range(100, 120)), list(range(100, 120))
        row_a = torch.full((16,), -1, dtype=torch.int32)
        row_a[:(L0 + ps - 1) // ps] = torch.arange(50, 50 + (L0 + ps - 1) // ps, dtype=torch.int32)
        row_b = row_a.clone()
        slots, L = oracle.store.append_chunk_paged(row_a, L0, rows, free_a, ps, 256)
        one_by_one = []
        lens = [L0]
        tab_b = row_b.view(1, -1)
        for _ in range(rows):
            one_by_one += oracle.store.append_token_paged(tab_b, lens, free_b, ps, 256, 10 ** 6)
        assert slots == one_by_one and L == lens[0] == L0 + rows
        assert torch.equal(row_a, row_b) and free_a == free_b
        assert 20 - len(free_a) == -(-(L0 + rows) // ps) - (-(-L0 // ps))     # closed form
    # two pages left for a chunk that wants three; the table ends at 40 tokens
    row = torch.full((4,), -1, dtype=torch.int32)
    slots, L = oracle.store.append_chunk_paged(row, 0, 48, [3, 9], ps, 64)
    assert L == 32 and slots[:16] == list(range(9 * 16, 10 * 16)) and slots[16:] == list(range(48, 64))
    row = torch.full((4,), -1, dtype=torch.int32)
    assert oracle.store.append_chunk_paged(row, 0, 48, [1, 2, 3, 4], ps, 40)[1] == 40
    # a full table or an empty stack leaves a request untouched
    t = torch.full((2, 2), -1, dtype=torch.int32)
    lens = [32, 16]
    assert oracle.store.append_token_paged(t, lens, [], ps, 32, 10 ** 6) == [None, None]
    assert lens == [32, 16] and bool((t == -1).all())
