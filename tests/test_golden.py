"""The committed golden fixture (tests/golden/decode_layer_small.npz, written by
tests/golden/make_fixtures.py from this repository's oracle): the oracle must
still reproduce it (CPU), and the HIP path must match it (GPU)."""

import os

import numpy as np
import pytest
import torch

import oracle

FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "decode_layer_small.npz")


def load():
    z = np.load(FIXTURE, allow_pickle=False)
    H, HKV, D, n_init, n_local, top_k, page = [int(x) for x in z["meta"]]
    bf = lambda name: torch.from_numpy(z[name].copy()).view(torch.bfloat16)
    return dict(z=z, H=H, HKV=HKV, D=D, n_init=n_init, n_local=n_local, top_k=top_k, page=page,
                rope_base=float(z["rope_base"][0]), seq_lens=[int(x) for x in z["seq_lens"]],
                table=torch.from_numpy(z["table"].copy()), k_pool=bf("k_pool"), v_pool=bf("v_pool"),
                q=bf("q"), out=bf("out"))


def test_oracle_reproduces_the_fixture():
    f = load()
    tabs = [oracle.select.expand_page_table(f["table"][b], L, f["page"])
            for b, L in enumerate(f["seq_lens"])]
    details = []
    sels, out = oracle.layer.decode_layer(
        f["q"], f["k_pool"], f["v_pool"], tabs, f["seq_lens"], f["H"], f["D"], f["n_init"],
        f["n_local"], [f["top_k"]] * len(tabs), f["rope_base"], 1.0, f["D"] ** -0.5, details=details)
    for b, sel in enumerate(sels):
        assert sel.tolist() == f["z"][f"sel_{b}"].tolist()
        if details[b]:
            assert np.allclose(details[b]["scores"].numpy(), f["z"][f"scores_{b}"], rtol=1e-5, atol=1e-4)
            assert details[b]["top_pos"].tolist() == f["z"][f"top_pos_{b}"].tolist()
    assert (out.float() - f["out"].float()).abs().max().item() <= 1e-2
    assert "sel_1" in f["z"] and "top_pos_1" not in f["z"]      # request 1 is the dense case
    assert f["z"]["sel_1"].shape[0] == f["seq_lens"][1]


@pytest.mark.gpu
def test_hip_path_matches_the_fixture(dev):
    from tokenselect_amd import ops
    f = load()
    B = len(f["seq_lens"])
    cfg = ops.LayerConfig(num_heads=f["H"], num_kv_heads=f["HKV"], page_size=f["page"],
                          n_init=f["n_init"], n_local=f["n_local"], top_k=f["top_k"],
                          rope_theta=f["rope_base"])
    bt = ops.Batch(torch.tensor(f["seq_lens"], dtype=torch.int32, device=dev),
                   f["table"].to(dev).contiguous(), max(f["seq_lens"]))
    layer = ops.DecodeLayer(cfg, B, max(f["seq_lens"]), dev)
    out, sel, sel_pos, sel_len = layer(f["q"].to(dev), f["k_pool"].to(dev), f["v_pool"].to(dev), bt)
    torch.cuda.synchronize()
    for b in range(B):
        want = f["z"][f"sel_{b}"]
        assert int(sel_len[b]) == want.shape[0]
        assert sel[b, :want.shape[0]].cpu().tolist() == want.tolist()
    assert (out.cpu().float() - f["out"].float()).abs().max().item() <= 2e-2


PREFILL_FIXTURE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "prefill_small.npz")


def load_prefill():
    z = np.load(PREFILL_FIXTURE, allow_pickle=False)
    names = ("H", "HKV", "D", "n_init", "n_local", "top_k", "L0", "T", "chunk")
    f = dict(zip(names, (int(x) for x in z["meta"])))
    bf = lambda name: torch.from_numpy(z[name].copy()).view(torch.bfloat16)
    f.update(z=z, rope_base=float(z["rope_base"][0]), k_pool=bf("k_pool"), v_pool=bf("v_pool"),
             table=torch.from_numpy(z["table"].copy()), new_slots=torch.from_numpy(z["new_slots"].copy()),
             q=bf("q"), k_new=bf("k_new"), v_new=bf("v_new"), out=bf("out"))
    return f


def test_oracle_reproduces_the_prefill_fixture():
    f = load_prefill()
    rows = f["L0"] + f["T"]
    tab = torch.zeros(rows, dtype=torch.int32)
    tab[:f["L0"]] = f["table"]
    details = []
    out = oracle.prefill.prefill(f["q"], f["k_new"], f["v_new"], f["k_pool"].clone(), f["v_pool"].clone(),
                                 tab, f["L0"], f["new_slots"], f["H"], f["D"], f["n_init"], f["n_local"],
                                 f["top_k"], f["rope_base"], 1.0, f["D"] ** -0.5, chunk=f["chunk"],
                                 details=details)
    assert len(details) == 3                                    # 32 + 32 + 6 rows
    for i, d in enumerate(details):
        assert d["top_pos"].tolist() == f["z"][f"top_pos_{i}"].tolist()
        assert torch.equal(d["qf"].view(torch.int16), torch.from_numpy(f["z"][f"qf_{i}"].copy()))
    assert (out.float() - f["out"].float()).abs().max().item() <= 1e-2


@pytest.mark.gpu
def test_hip_prefill_matches_the_fixture(dev):
    """Chunk by chunk: device fingerprint within one bf16 ulp of the fixture's; every
    chunk's selection and output against the oracle following the device's fingerprint;
    and, wherever the fingerprints agree bit for bit, against the fixture itself."""
    from tokenselect_amd import ops
    from helpers import assert_index_sets_match
    f = load_prefill()
    H, D, L0, T, chunk = f["H"], f["D"], f["L0"], f["T"], f["chunk"]
    cfg = ops.LayerConfig(num_heads=H, num_kv_heads=f["HKV"], n_init=f["n_init"], n_local=f["n_local"],
                          top_k=f["top_k"], rope_theta=f["rope_base"])
    k_pool, v_pool = f["k_pool"].to(dev), f["v_pool"].to(dev)
    table = torch.zeros((1, L0 + T), dtype=torch.int32, device=dev)
    table[0, :L0] = f["table"].to(dev)
    seq = torch.tensor([L0], dtype=torch.int32, device=dev)
    layer = ops.PrefillChunk(cfg, L0 + T, dev, max_rows=chunk)
    kc, vc = f["k_pool"].clone(), f["v_pool"].clone()
    tab_cpu = torch.zeros(L0 + T, dtype=torch.int32)
    tab_cpu[:L0] = f["table"]
    q, L = f["q"].to(dev), L0
    for i, start in enumerate(range(0, T, chunk)):
        end = min(start + chunk, T)
        m = end - start
        ops.kv_store_chunk(cfg, f["k_new"][start:end].to(dev), f["v_new"][start:end].to(dev),
                           f["new_slots"][start:end].to(dev).contiguous(), k_pool, v_pool, table[0], seq)
        L += m
        out, sel, sel_pos, sel_len = layer(q[start:end].contiguous(), k_pool, v_pool,
                                           ops.Batch(seq, table, L))
        qf = ops.fingerprint(cfg, q[start:end].view(m, H, D).contiguous(), layer.cos, layer.sin)
        torch.cuda.synchronize()
        want_qf = torch.from_numpy(f["z"][f"qf_{i}"].copy()).view(torch.bfloat16).float()
        got_qf = qf.cpu().float().reshape(-1)
        assert bool(((got_qf - want_qf).abs() <= want_qf.abs() * 2.0 ** -7 + 1e-30).all())
        S = int(sel_len[0])
        assert S == f["n_init"] + f["top_k"] + f["n_local"]
        # the oracle on the same pools, with the device's fingerprint
        loc = f["new_slots"][start:end].long()
        kc[loc], vc[loc] = f["k_new"][start:end], f["v_new"][start:end]
        tab_cpu[L - m:L] = f["new_slots"][start:end].to(torch.int32)
        d = {}
        ref_slots, ref_out = oracle.prefill.prefill_chunk(
            f["q"][start:end], kc, vc, tab_cpu, L, H, D, f["n_init"], f["n_local"], f["top_k"],
            f["rope_base"], 1.0, D ** -0.5, detail=d, qf_override=qf.cpu())
        mid = sel_pos[0, f["n_init"]:f["n_init"] + f["top_k"]].cpu()
        assert_index_sets_match(mid, d["top_pos"], d["votes"], f["n_init"], f"fixture chunk {i}")
        got_slots = sel[0, :S].cpu()
        if not torch.equal(got_slots, ref_slots):               # a tie went the other way
            ref_out = oracle.prefill.sparse_prefill_attention(
                f["q"][start:end].view(m, H, D), kc, vc, got_slots, D ** -0.5,
                f["rope_base"]).reshape(m, -1)
        assert (out.cpu().float() - ref_out.float()).abs().max().item() <= 2e-2, f"chunk {i}"
        if torch.equal(got_qf, want_qf) and mid.tolist() == f["z"][f"top_pos_{i}"].tolist():
            assert (out.cpu().float() - f["out"][start:end].float()).abs().max().item() <= 2e-2
