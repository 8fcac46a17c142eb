"""The Llama-shaped decoder around the TokenSelect layer, at toy size: every layer's
library call against the CPU oracle on the very query and pools it saw (slots
identical up to ties at the k-th vote, attention within 2e-2), the store + table
append of every layer, and the logits against a plain CPU restatement of the
whole forward."""

import pytest
import torch
import torch.nn.functional as F

import oracle
from tokenselect_amd.model import Decoder, ModelConfig
from helpers import assert_index_sets_match, say

pytestmark = pytest.mark.gpu

TOY = dict(layers=3, hidden=256, intermediate=384, vocab=500, num_heads=8, num_kv_heads=2,
           rope_theta=1e4, n_init=4, n_local=16, top_k=32, init_std=0.05)


# Votes this close (relative) to the k-th one count as tied with it in the whole-forward check:
# there the oracle selects with its own query, which differs from the device's by the bf16
# rounding of the layers before (1e-2 absolute), and that moves a vote by up to a few percent.
NEAR_TIE = 5e-2


def _cpu_forward(m: Decoder, tokens, kc, vc, tab, lens, loc, device_sels):
    """fp32 restatement of Decoder.decode_step on CPU copies of the cache (updated in
    place), intermediates rounded to bf16 where the device rounds them.  Where a layer's
    selection differs from the device's (``device_sels[l]``: slots and counts) only in members
    whose vote is within NEAR_TIE of the k-th vote, the attention follows the device's slots:
    one swapped token changes the output by far more than any rounding does.  (The exact
    comparison of every layer's selection, on the device's own query, is the caller's.)"""
    mc, c = m.mc, m.cfg
    bf = lambda t: t.bfloat16().float()
    norm = lambda x, w: bf(F.rms_norm(x, (mc.hidden,), w.cpu().float(), mc.rms_eps))
    hd, kvd = mc.num_heads * mc.head_dim, mc.num_kv_heads * mc.head_dim
    x = m.embed.cpu().float()[tokens]
    for l in range(mc.layers):
        qkv = bf(norm(x, m.norm_in[l]) @ m.wqkv[l].cpu().float().T)
        q, k, v = qkv.split((hd, kvd, kvd), dim=-1)
        for b in range(m.batch):
            kc[l][loc[b]] = k[b].view(mc.num_kv_heads, mc.head_dim).bfloat16()
            vc[l][loc[b]] = v[b].view(mc.num_kv_heads, mc.head_dim).bfloat16()
        d = []
        sels, attn = oracle.layer.decode_layer(
            q.bfloat16(), kc[l], vc[l], [tab[b] for b in range(m.batch)], lens, mc.num_heads,
            mc.head_dim, c.n_init, c.n_local, [c.top_k] * m.batch, c.rope_theta, c.rope_scale,
            mc.head_dim ** -0.5, details=d)
        for b in range(m.batch):
            got = device_sels[l][0][b, :int(device_sels[l][1][b])].cpu()
            if torch.equal(got, sels[b]):
                continue
            inv = {int(s): p for p, s in enumerate(tab[b, :lens[b]].tolist())}
            pos = torch.tensor([inv[int(s)] for s in got.tolist()])
            assert_index_sets_match(pos[c.n_init:c.n_init + c.top_k], d[b]["top_pos"], d[b]["votes"],
                                    c.n_init, f"whole forward, layer {l} request {b}", rtol=NEAR_TIE)
            attn[b] = oracle.attend.sparse_decode_attention(
                q[b].bfloat16().view(mc.num_heads, mc.head_dim), kc[l], vc[l], got, mc.head_dim ** -0.5,
                c.rope_theta, c.rope_scale).reshape(-1)
        x = bf(x + bf(attn.float() @ m.wo[l].cpu().float().T))
        gate, up = bf(norm(x, m.norm_post[l]) @ m.w_gate_up[l].cpu().float().T).chunk(2, dim=-1)
        x = bf(x + bf(bf(bf(F.silu(gate)) * up) @ m.w_down[l].cpu().float().T))
    return norm(x, m.final_norm) @ m.lm_head.cpu().float().T


@pytest.mark.parametrize("query_cache,fused_qkv", [(False, True), (False, False), (True, True), (True, False)],
                         ids=["plain", "plain-gemm-then-store", "query_cache", "query_cache-gemm-then-store"])
def test_decoder_steps_match_the_oracle(dev, query_cache, fused_qkv):
    say(f"toy decoder, query_cache={query_cache} fused_qkv={fused_qkv}")
    mc = ModelConfig(**TOY)
    contexts, steps = [300, 41], 3          # the second request attends densely
    m = Decoder(mc, contexts, steps, dev, seed=21, query_cache=query_cache, fused_qkv=fused_qkv)
    assert m.fused_qkv == fused_qkv
    c = m.cfg
    kc = [p.cpu().clone() for p in m.k_pools]
    vc = [p.cpu().clone() for p in m.v_pools]
    tab = m.table.cpu().clone()
    tokens = torch.tensor([7, 123], device=dev)
    for t in range(steps):
        trace = []
        logits = m.decode_step(tokens, trace)
        torch.cuda.synchronize()
        lens = [L + t + 1 for L in contexts]
        loc = m.free[t].cpu().long()
        for b in range(m.batch):
            tab[b, lens[b] - 1] = loc[b]
        assert torch.equal(m.table.cpu(), tab)
        assert m.num_tokens.cpu().tolist() == [lens] * mc.layers

        if not query_cache:   # with the cache on, a hit legitimately reuses older positions
            ref = _cpu_forward(m, tokens.cpu(), kc, vc, tab, lens, loc,
                               [(sel, sel_len) for (_, _, _, _, sel, sel_len) in trace])
            scale = ref.pow(2).mean().sqrt().item()
            err = (logits.cpu().float() - ref).abs().max().item()
            assert err <= 0.05 * scale, (t, err, scale)

        # every layer's call, on the query and the pools the device used
        for l, (q, k, v, attn, sel, sel_len) in enumerate(trace):
            kl, vl = m.k_pools[l].cpu(), m.v_pools[l].cpu()
            assert torch.equal(kl[loc], k.cpu().view(m.batch, mc.num_kv_heads, mc.head_dim))
            assert torch.equal(vl[loc], v.cpu().view(m.batch, mc.num_kv_heads, mc.head_dim))
            d = []
            if query_cache and t > 0:
                continue
            ref_sels, ref_out = oracle.layer.decode_layer(
                q.cpu(), kl, vl, [tab[b] for b in range(m.batch)], lens, mc.num_heads, mc.head_dim,
                c.n_init, c.n_local, [c.top_k] * m.batch, c.rope_theta, c.rope_scale,
                mc.head_dim ** -0.5, details=d)
            for b in range(m.batch):
                S = int(sel_len[b])
                assert S == ref_sels[b].shape[0]
                got = sel[b, :S].cpu()
                if "top_pos" in d[b]:
                    inv = {int(s): p for p, s in enumerate(tab[b, :lens[b]].tolist())}
                    pos = torch.tensor([inv[int(s)] for s in got.tolist()])
                    assert_index_sets_match(pos[c.n_init:c.n_init + c.top_k], d[b]["top_pos"],
                                            d[b]["votes"], c.n_init, f"step {t} layer {l} request {b}")
                else:
                    assert torch.equal(got, ref_sels[b])
                want = ref_out[b]
                if not torch.equal(got, ref_sels[b]):   # a tie went the other way: follow the device's slots
                    want = oracle.attend.sparse_decode_attention(
                        q.cpu()[b].view(mc.num_heads, mc.head_dim), kl, vl, got, mc.head_dim ** -0.5,
                        c.rope_theta, c.rope_scale).reshape(-1)
                err = (attn[b].cpu().float().reshape(-1) - want.float()).abs().max().item()
                assert err <= 2e-2, (t, l, b, err)
        tokens = logits.argmax(dim=-1)
    if query_cache:
        lookups = sum(int(cache.counters[:, 1].sum()) for cache in m.caches)
        assert lookups == mc.layers * steps        # only the long request consults its cache


def test_generate_is_deterministic_and_bounded(dev):
    say("toy decoder, greedy generation")
    mc = ModelConfig(**TOY)
    runs = []
    for _ in range(2):
        m = Decoder(mc, [200, 150], 4, dev, seed=5)
        runs.append(m.generate(torch.tensor([1, 2], device=dev), 4).cpu())
    assert torch.equal(runs[0], runs[1])
    with pytest.raises(RuntimeError, match="no slot left"):
        m.decode_step(torch.tensor([1, 2], device=dev))


def test_a_step_that_gave_up_is_redone_where_the_tokens_are_read_back(dev):
    """A fused selection that gives up in the middle of a decode step (forced from the host:
    an absent team member and a 20 us bound, every kernel still exits) is noticed where the
    step's tokens reach the host; the step is undone and repeated with the separate kernels,
    and the tokens, logits, tables and lengths equal those of an undisturbed model."""
    say("toy decoder, a decode step that gave up and is redone")
    mc = ModelConfig(**TOY)
    contexts, steps, bad = [300, 260], 4, 1
    runs = []
    for disturb in (False, True):
        m = Decoder(mc, contexts, steps, dev, seed=33)
        tokens = torch.tensor([7, 123], device=dev)
        out = []
        for t in range(steps):
            if disturb and t == bad:
                m.layer_options = dict(wait_us=20, absent_workgroups=1)
            logits, tokens, host = m.decode_step_checked(tokens)
            out.append((logits.float().cpu(), host.clone()))
        torch.cuda.synchronize()
        assert m.steps_redone == (1 if disturb else 0)
        assert m.attention.separate == disturb
        runs.append((out, m.table.cpu(), m.num_tokens.cpu()))
    (plain, tab0, n0), (redone, tab1, n1) = runs
    assert torch.equal(tab0, tab1) and torch.equal(n0, n1)
    assert n0.tolist() == [[c + steps for c in contexts]] * mc.layers
    for t in range(steps):
        scale = plain[t][0].pow(2).mean().sqrt().item()
        assert (plain[t][0] - redone[t][0]).abs().max().item() <= 0.02 * scale, t
        assert torch.equal(plain[t][1], redone[t][1]), f"step {t}: tokens differ"
