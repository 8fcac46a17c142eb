"""The decode layer under HIP graph capture, the way a serving stack replays a decode step:
`ts_decode_layer` only launches kernels (its side jobs, clearing counters and tickets, are
kernels too), so a captured call replays with new queries, new lengths and new table
contents in the same buffers.  Every replay is checked against an eager call of a second
layer object on the same inputs, with eager work and synchronisations in between."""

import pytest
import torch

from helpers import say
from tokenselect_amd import ops, workloads

pytestmark = pytest.mark.gpu

SHAPE = dict(num_heads=32, num_kv_heads=8, rope_theta=5e5)


@pytest.fixture
def fused_select(request):
    previous = ops.set_fused_select(request.param)
    yield request.param
    ops.set_fused_select(previous)


def _capture(layer, q, k_pool, v_pool, bt):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # the first calls load code objects and size the grids
        for _ in range(2):
            layer(q, k_pool, v_pool, bt)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outputs = layer(q, k_pool, v_pool, bt)
    return graph, outputs


@pytest.mark.parametrize("fused_select", [True, False], indirect=True, ids=["fused", "separate"])
@pytest.mark.parametrize("pool_kernel", [-1, 5], ids=["plain", "max-pool"])
def test_decode_layer_replays_in_a_graph(dev, fused_select, pool_kernel):
    lens, ks = [5000, 100, 2048, 901], [256, 256, 200, 256]
    say(f"decode_layer in a graph: fused={fused_select} pool_kernel={pool_kernel}")
    wl = workloads.build("small", SHAPE, lens, ks, 16, dev, 61, n_init=16, n_local=32, top_k=256,
                         pool_kernel=pool_kernel)
    c, bt = wl.cfg, wl.batch
    q = wl.q.clone()
    layer = ops.DecodeLayer(c, len(lens), max(lens), dev)
    eager = ops.DecodeLayer(c, len(lens), max(lens), dev)
    graph, (out, sel, sel_pos, sel_len) = _capture(layer, q, wl.k_pool, wl.v_pool, bt)
    gen = torch.Generator(device=dev).manual_seed(62)
    for replay in range(5):
        # new inputs in the captured buffers: another query, shorter contexts from the
        # third replay on (a request of 100 tokens stays dense), new keys in the pool
        q.copy_(torch.randn(q.shape, device=dev, generator=gen).to(q.dtype))
        if replay >= 2:
            bt.seq_lens.sub_(torch.tensor([37, 0, 5, 1], dtype=torch.int32, device=dev))
        if replay == 3:
            wl.k_pool[::7].mul_(-1)
        graph.replay()
        torch.cuda.synchronize()
        layer.check()
        got = [t.clone() for t in (out, sel, sel_pos, sel_len)]
        want = eager(q, wl.k_pool, wl.v_pool, bt)
        torch.cuda.synchronize()
        assert torch.equal(got[3], want[3]), f"replay {replay}: lengths"
        for b in range(len(lens)):
            S = int(want[3][b])
            assert torch.equal(got[2][b, :S], want[2][b, :S]), f"replay {replay} b={b}: positions"
            assert torch.equal(got[1][b, :S], want[1][b, :S]), f"replay {replay} b={b}: slots"
        assert torch.equal(got[0].view(torch.int16), want[0].view(torch.int16)), f"replay {replay}: out"
    # and the replays moved with their inputs: the last lengths are the shortened ones
    assert sel_len.tolist() == [16 + 256 + 32, 100, 16 + 200 + 32, 16 + 256 + 32]
