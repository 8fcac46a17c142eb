"""``ts_sparse_decode_attn_static``, the entry point that allocates nothing (its
split-K partials live in a buffer built into the library), against
``ts_sparse_decode_attn`` with a caller's workspace: same kernels, so the outputs
must be bit-identical.  Two calls in a row share the built-in buffer, the second
with a smaller input (fewer requests, shorter lists, another split count)."""

import ctypes

import pytest
import torch

import oracle
from tokenselect_amd import _lib, ops, workloads
from helpers import say

pytestmark = pytest.mark.gpu


def _case(dev, seed, lens, width):
    wl = workloads.build("static-attn", workloads.LLAMA3_8B, [4000] * len(lens), [64] * len(lens), 1,
                         dev, seed, n_init=8, n_local=16)
    g = torch.Generator().manual_seed(seed)
    sel = torch.zeros((len(lens), width), dtype=torch.int32)
    for b, S in enumerate(lens):
        sel[b, :S] = torch.randperm(wl.k_pool.shape[0], generator=g)[:S].int()
    return wl, sel, torch.tensor(lens, dtype=torch.int32)


def test_static_scratch_matches_the_workspace_entry_point(dev):
    lib = _lib.load()
    assert lib.ts_attn_static_scratch_bytes() == 4 << 20
    # first call: 3 requests, up to 2688 selected; second call: 1 request, 300 selected
    for seed, lens, width in [(21, [2688, 1500, 40], 2688), (22, [300], 300)]:
        say(f"static-scratch attention lens={lens}")
        wl, sel, sel_len = _case(dev, seed, lens, width)
        c = wl.cfg
        sel_d, len_d = sel.to(dev), sel_len.to(dev)
        want = ops.sparse_decode_attention(c, wl.q, wl.k_pool, wl.v_pool, sel_d, len_d)
        out = torch.full_like(want, float("nan"))
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
        code = lib.ts_sparse_decode_attn_static(
            ctypes.byref(c.to_c()), wl.q.data_ptr(), wl.k_pool.data_ptr(), wl.v_pool.data_ptr(),
            wl.k_pool.shape[0], sel_d.data_ptr(), sel_d.stride(0), len_d.data_ptr(), len(lens), width,
            out.data_ptr(), torch.cuda.current_stream().cuda_stream)
        assert code == _lib.TS_OK, lib.ts_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before
        assert torch.equal(out.view(torch.int16), want.view(torch.int16)), \
            f"lens={lens}: max |diff| {(out.float() - want.float()).abs().max().item()}"
        # and both agree with the oracle on the first request
        ref = oracle.attend.sparse_decode_attention(
            wl.q.cpu()[0].view(c.num_heads, 128), wl.k_pool.cpu(), wl.v_pool.cpu(), sel[0, :lens[0]],
            128 ** -0.5, c.rope_theta, 1.0, 0.0, c.rope_mode)
        assert (out[0].cpu().float() - ref.reshape(-1).float()).abs().max().item() <= 2e-2


def test_static_scratch_call_replays_in_a_graph(dev):
    """What the entry point is for: captured into a HIP graph (the buffer's address was looked
    up at set-up, the tickets are cleared by a kernel, nothing allocates) and replayed with new
    queries, lists and lengths in the captured buffers; every replay, with eager work and
    synchronisations in between, equals an eager call with a caller's workspace."""
    lib = _lib.load()
    assert lib.ts_attn_static_scratch_bytes() == 4 << 20      # set-up: resolves the buffer
    lens, width = [2688, 1500, 40], 2688
    say(f"static-scratch attention in a graph lens={lens}")
    wl, sel, sel_len = _case(dev, 23, lens, width)
    c = wl.cfg
    q, sel_d, len_d = wl.q.clone(), sel.to(dev), sel_len.to(dev)
    out = torch.zeros_like(q)

    def call():
        code = lib.ts_sparse_decode_attn_static(
            ctypes.byref(c.to_c()), q.data_ptr(), wl.k_pool.data_ptr(), wl.v_pool.data_ptr(),
            wl.k_pool.shape[0], sel_d.data_ptr(), sel_d.stride(0), len_d.data_ptr(), len(lens), width,
            out.data_ptr(), torch.cuda.current_stream().cuda_stream)
        assert code == _lib.TS_OK, lib.ts_last_error()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):      # loads the code object before the capture
        call()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    gen = torch.Generator(device=dev).manual_seed(24)
    for replay in range(4):
        q.copy_(torch.randn(q.shape, device=dev, generator=gen).to(q.dtype))
        if replay >= 2:   # shorter lists, other slots
            len_d.copy_(torch.tensor([900, 1500 - replay, 17], dtype=torch.int32))
            sel_d.copy_(sel_d.flip(1))
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = ops.sparse_decode_attention(c, q, wl.k_pool, wl.v_pool, sel_d, len_d)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"replay {replay}"
