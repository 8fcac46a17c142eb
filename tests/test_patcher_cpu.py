"""Host logic of the patch-layer mirror, without a GPU: the reference's entry
point names, signatures and defaults (tr.py:885-894, 117-129, 234-244, 264-277),
the globals ``patch()`` sets (tr.py:895-918), the token-table bookkeeping
(tr.py:324-336) and the error / sentinel behaviour (tr.py:334, 377-378, 650)."""

import inspect

import pytest
import torch

from tokenselect_amd.patcher import sglang_standins as sg
from tokenselect_amd.patcher import token_retrieval as tr


def params(fn):
    return [(n, p.default) for n, p in inspect.signature(fn).parameters.items()
            if p.kind is not inspect.Parameter.KEYWORD_ONLY]


def test_signatures_match_the_reference():
    E = inspect.Parameter.empty
    assert params(tr.patch) == [("rope_base", 1e6), ("rope_scale", 1), ("rope_model", "ROPE_LLAMA"),
                                ("max_n_tokens", 1024), ("top_k", 16), ("n_init", 1),
                                ("n_local", 16), ("kernel_size", -1)]
    assert [n for n, _ in params(tr.ReqToTokenRetriever.__init__)] == [
        "self", "num_layers", "head_dim", "num_heads", "num_kv_heads", "fingerprint_dim",
        "max_num_tokens", "token_to_kv_pool", "dtype", "device"]
    assert params(tr.TokenRetriever.__init__) == [
        ("self", E), ("num_layers", E), ("head_dim", E), ("num_heads", E), ("num_kv_heads", E),
        ("fingerprint_dim", E), ("max_num_tokens", E), ("dtype", E), ("device", E),
        ("token_to_kv_pool", None), ("rotary_embedding", None)]
    assert params(tr.paged_matmul) == [
        ("query", E), ("token", E), ("indices", E), ("scores", E), ("num_relevant_tokens", E),
        ("num_heads", E), ("num_kv_heads", E), ("head_dim", E), ("BLOCK_SIZE_TOKENS", 128)]
    assert params(tr.RotaryEmbedding.__init__) == [("self", E), ("dim", E), ("base", E),
                                                   ("distance_scale", 1.0), ("device", "cuda")]
    assert [n for n, _ in params(tr.TokenRetriever.retrieval_indices)] == [
        "self", "query", "layer_id", "n_init", "n_local", "topk"]
    assert [n for n, _ in params(tr.TokenRetriever.get_topk_tokens)] == [
        "self", "query_fingerprints", "token_fingerprints", "topk", "indices"]
    assert params(tr.patched_radix_attention_store_kv_cache)[-2:] == [("start", 0), ("end", None)]
    for name in ("patched_radix_attention_forward", "patched_radix_attention_decode_forward_flashinfer",
                 "patched_radix_attention_extend_forward_flashinfer"):
        assert [n for n, _ in params(getattr(tr, name))] == ["self", "q", "k", "v", "input_metadata"]
    assert [n for n, _ in params(tr.patched_meta_attention_forward)] == [
        "self", "positions", "hidden_states", "input_metadata"]
    for name in ("patch_model_runner", "patch_input_metadata", "patch_model", "cuda_timer"):
        assert callable(getattr(tr, name))


def test_patch_sets_the_reference_globals_and_patches_the_classes():
    tr.patch(rope_base=500000, rope_scale=1, rope_model="ROPE_LLAMA", max_n_tokens=1048576,
             n_init=128, n_local=512, top_k=2048)
    assert (tr.ROPE_BASE, tr.ROPE_SCALE, tr.ROPE_MODE) == (500000, 1, "ROPE_LLAMA")
    assert (tr.MAX_N_TOKENS, tr.TOP_K, tr.N_INIT, tr.N_Local, tr.KERNEL_SIZE) == (1048576, 2048, 128,
                                                                                 512, -1)
    # hard-coded by the reference, tr.py:916-918
    assert tr.QUERY_ROTATE is True and tr.PREFILL_CHUNK_SIZE == 512 and tr.QUERY_CACHE is False
    assert sg.RadixAttention.forward is tr.patched_radix_attention_forward
    assert sg.RadixAttention.store_kv_cache is tr.patched_radix_attention_store_kv_cache
    assert sg.Attention.forward is tr.patched_meta_attention_forward
    tr.patch(query_cache=True)
    assert tr.QUERY_CACHE is True and tr.TOP_K == 16 and tr.N_Local == 16
    tr.patch()


def make_retriever(layers=2, max_tokens=64):
    tr.patch(rope_base=1e4, top_k=8, n_init=2, n_local=4, max_n_tokens=max_tokens)
    pool = sg.TokenToKVPool(128, torch.bfloat16, 2, 128, layers, "cpu")
    req = tr.ReqToTokenRetriever(layers, 128, 4, 2, 256, max_tokens, pool, torch.bfloat16, "cpu")
    return req, pool


def test_token_table_bookkeeping():
    req, pool = make_retriever()
    r = req.get_token_retriever("a")
    assert r is req.get_token_retriever("a")                 # same request -> same retriever
    assert r.token_fingerprints[1] is pool.get_key_buffer(1)  # aliased, not copied
    assert r.token_indices.shape == (2, 64) and r.token_indices.dtype == torch.int32
    r.add_k_cache(torch.tensor([5, 9, 2], dtype=torch.int32), 0)
    r.add_k_cache(torch.tensor([7], dtype=torch.int32), 0)
    assert r.num_tokens == [4, 0]
    assert r.get_all_tokens(0).tolist() == [5, 9, 2, 7] and r.get_all_tokens(1).tolist() == []
    with pytest.raises(AssertionError):
        r.add_k_cache(torch.zeros(61, dtype=torch.int32), 0)  # tr.py:334
    r2 = req.get_token_retriever("b")                         # new request -> fresh state
    assert r2 is not r and r2.num_tokens == [0, 0] and r2.is_first_query == [True, True]
    r.clear()
    assert r.num_tokens == [0, 0]


def test_short_context_returns_none_without_touching_the_gpu():
    req, _ = make_retriever()
    r = req.get_token_retriever("a")
    r.add_k_cache(torch.arange(14, dtype=torch.int32), 0)
    q = torch.zeros(1, 4 * 128, dtype=torch.bfloat16)
    assert r.retrieval_indices(q, 0, 2, 4, 8) is None         # 2 + 8 + 4 >= 14, tr.py:377-378
    r.add_k_cache(torch.tensor([14], dtype=torch.int32), 0)
    with pytest.raises(ValueError, match="no CPU path"):      # 15 tokens: selection needs the GPU
        r.retrieval_indices(q, 0, 2, 4, 8)


def test_forward_dispatch_and_unsupported_modes():
    tr.patch(rope_base=1e4, top_k=8, n_init=2, n_local=4, max_n_tokens=64)
    attn = sg.RadixAttention(4, 128, 128 ** -0.5, 2, layer_id=0)
    meta = sg.InputMetadata(sg.ForwardMode.PREFILL, None, None, torch.zeros(1, dtype=torch.int32))
    q = torch.zeros(1, 4 * 128, dtype=torch.bfloat16)
    assert attn.forward(q, None, None, meta) is None          # neither EXTEND nor DECODE, tr.py:835-842
    sliding = sg.RadixAttention(4, 128, 128 ** -0.5, 2, layer_id=0, sliding_window_size=4096)
    for mode in (sg.ForwardMode.EXTEND, sg.ForwardMode.DECODE):
        meta.forward_mode = mode
        with pytest.raises(NotImplementedError, match="Sliding window"):
            sliding.forward(q, None, None, meta)
    meta.forward_mode = sg.ForwardMode.DECODE
    with pytest.raises(AssertionError):                       # k without v, tr.py:830-831
        attn.forward(q, torch.zeros(1, 256, dtype=torch.bfloat16), None, meta)


def test_rotary_tables_follow_the_reference_expressions():
    rot = tr.RotaryEmbedding(128, 5e5, 1.0, device="cpu")
    rot._update_cos_sin_tables(600)
    assert rot._cos_table.shape == (600, 1, 128) and rot._cos_table.dtype == torch.float32
    inv = 1.0 / (5e5 ** (torch.arange(0, 128, 2, dtype=torch.float32) / 128))
    ang = 512 * inv
    assert torch.equal(rot._cos_table[512, 0, :64], ang.cos())
    assert torch.equal(rot._sin_table[512, 0, 64:], ang.sin())
    x = torch.arange(8.0).view(1, 8)
    assert rot.rotate_half(x).tolist() == [[-4.0, -5.0, -6.0, -7.0, 0.0, 1.0, 2.0, 3.0]]
