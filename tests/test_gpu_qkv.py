"""The QKV projection with the KV store as its epilogue (ts_qkv_store) against an fp64
product of the same bf16 operands (within one bf16 ulp of the exact value), and its
store / append semantics against ts_kv_store's."""

import pytest
import torch

from tokenselect_amd import ops
from helpers import say

pytestmark = pytest.mark.gpu

CASES = [
    dict(num_heads=32, num_kv_heads=8, hidden=4096, batch=4, bias=False),   # Llama-3-8B
    dict(num_heads=32, num_kv_heads=8, hidden=4096, batch=8, bias=False),   # 64 KB of x in LDS
    dict(num_heads=28, num_kv_heads=4, hidden=3584, batch=1, bias=True),    # Qwen2-7B
    dict(num_heads=28, num_kv_heads=4, hidden=3584, batch=7, bias=True),
    dict(num_heads=4, num_kv_heads=2, hidden=264, batch=3, bias=True),      # ragged reduction split
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"H{c['num_heads']}kv{c['num_kv_heads']}h{c['hidden']}b{c['batch']}")
def test_qkv_store(dev, case):
    say(f"qkv_store {case}")
    H, Hkv, hidden, B = case["num_heads"], case["num_kv_heads"], case["hidden"], case["batch"]
    cfg = ops.LayerConfig(num_heads=H, num_kv_heads=Hkv, page_size=1)
    g = torch.Generator(device=dev).manual_seed(hidden + B)
    n_out = (H + 2 * Hkv) * 128
    x = torch.randn((B, hidden), generator=g, device=dev).bfloat16()
    w = (0.05 * torch.randn((n_out, hidden), generator=g, device=dev)).bfloat16()
    bias = torch.randn((n_out,), generator=g, device=dev).bfloat16() if case["bias"] else None
    rows, L0, max_tokens = 64, 20, 40
    k_pool = torch.randn((rows, Hkv, 128), generator=g, device=dev).bfloat16()
    v_pool = torch.randn((rows, Hkv, 128), generator=g, device=dev).bfloat16()
    k_before, v_before = k_pool.clone(), v_pool.clone()
    loc = torch.randperm(rows, generator=g, device=dev)[:B].int()
    table = torch.full((B, max_tokens), -1, dtype=torch.int32, device=dev)
    seq = torch.arange(L0, L0 + B, dtype=torch.int32, device=dev)
    assert ops.qkv_store_supported(B, hidden)
    q = ops.qkv_store(cfg, x, w, bias, loc, k_pool, v_pool, table, seq)
    torch.cuda.synchronize()

    ref = x.double() @ w.double().T
    if bias is not None:
        ref = ref + bias.double()
    got = torch.cat([q, k_pool[loc.long()].reshape(B, -1), v_pool[loc.long()].reshape(B, -1)], dim=1)
    # fp32 accumulation, then one rounding to bf16: half an ulp of rounding plus the
    # accumulation error, bounded here by one ulp of the exact value.
    ulp = ref.abs().clamp_min(2.0 ** -100) * 2.0 ** -8
    excess = ((got.double() - ref).abs() - ulp).max().item()
    assert excess <= 1e-6 * ref.abs().max().item(), excess
    assert (got.double() - ref).abs().max().item() > 0     # it did compute something

    untouched = torch.ones(rows, dtype=torch.bool, device=dev)
    untouched[loc.long()] = False
    assert torch.equal(k_pool[untouched], k_before[untouched])
    assert torch.equal(v_pool[untouched], v_before[untouched])
    for b in range(B):
        assert int(seq[b]) == L0 + b + 1
        assert int(table[b, L0 + b]) == int(loc[b])
        assert int((table[b] != -1).sum()) == 1


def test_qkv_store_matches_gemm_then_kv_store(dev):
    """Same state as the two-step path it replaces, up to the last bit of the bf16 rounding."""
    say("qkv_store vs linear + kv_store")
    H, Hkv, hidden, B = 8, 2, 512, 4
    cfg = ops.LayerConfig(num_heads=H, num_kv_heads=Hkv, page_size=1)
    g = torch.Generator(device=dev).manual_seed(3)
    n_out = (H + 2 * Hkv) * 128
    x = torch.randn((B, hidden), generator=g, device=dev).bfloat16()
    w = (0.05 * torch.randn((n_out, hidden), generator=g, device=dev)).bfloat16()
    loc = torch.tensor([5, 9, 2, 30], dtype=torch.int32, device=dev)
    pools = [torch.zeros((32, Hkv, 128), dtype=torch.bfloat16, device=dev) for _ in range(4)]
    tables = [torch.zeros((B, 16), dtype=torch.int32, device=dev) for _ in range(2)]
    seqs = [torch.full((B,), 7, dtype=torch.int32, device=dev) for _ in range(2)]
    q1 = ops.qkv_store(cfg, x, w, None, loc, pools[0], pools[1], tables[0], seqs[0])
    q2, k2, v2 = torch.nn.functional.linear(x, w).split((H * 128, Hkv * 128, Hkv * 128), dim=-1)
    ops.kv_store(cfg, k2.contiguous(), v2.contiguous(), loc, pools[2], pools[3], tables[1], seqs[1])
    torch.cuda.synchronize()
    assert torch.equal(tables[0], tables[1]) and torch.equal(seqs[0], seqs[1])
    for mine, theirs in ((q1, q2), (pools[0], pools[2]), (pools[1], pools[3])):
        diff = (mine.float() - theirs.float()).abs()
        assert bool((diff <= theirs.float().abs() * 2.0 ** -7 + 1e-30).all())


def test_qkv_store_full_table_and_limits(dev):
    say("qkv_store limits")
    H, Hkv, hidden = 4, 2, 256
    cfg = ops.LayerConfig(num_heads=H, num_kv_heads=Hkv, page_size=1)
    n_out = (H + 2 * Hkv) * 128
    w = torch.zeros((n_out, hidden), dtype=torch.bfloat16, device=dev)
    pool = torch.zeros((8, Hkv, 128), dtype=torch.bfloat16, device=dev)
    x = torch.zeros((2, hidden), dtype=torch.bfloat16, device=dev)
    loc = torch.tensor([1, 2], dtype=torch.int32, device=dev)
    table = torch.full((2, 4), -1, dtype=torch.int32, device=dev)
    seq = torch.tensor([4, 3], dtype=torch.int32, device=dev)      # request 0: table full
    ops.qkv_store(cfg, x, w, None, loc, pool, pool.clone(), table, seq)
    torch.cuda.synchronize()
    assert seq.tolist() == [4, 4]
    assert table[0].tolist() == [-1] * 4 and table[1].tolist() == [-1, -1, -1, 2]
    assert not ops.qkv_store_supported(9, hidden) and not ops.qkv_store_supported(2, 4100)
    big = torch.zeros((9, hidden), dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError):
        ops.qkv_store(cfg, big, w, None, torch.zeros(9, dtype=torch.int32, device=dev), pool,
                      pool.clone(), torch.zeros((9, 4), dtype=torch.int32, device=dev),
                      torch.zeros(9, dtype=torch.int32, device=dev))
