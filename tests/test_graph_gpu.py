"""The op-level entry points neither allocate nor synchronise, so a caller can capture them in a
HIP graph: the MoE layer and decode attention are captured once and replayed with new inputs, with
eager work and synchronisations between the replays; every replay must reproduce the eager result
bit for bit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_moe_layer_and_attention_replay_in_a_graph(ops):
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(5)

    def n(*shape, std=0.02):
        return (torch.randn(*shape, device=dev, generator=g) * std).to(torch.bfloat16)

    B, E, H, I = 200, 8, 256, 512
    layer = ops.MoeLayer(n(E, H), n(E), n(E, 2 * I, H), n(E, 2 * I), n(E, H, I), n(E, H), max_tokens=B)
    n_q, n_kv, D, S = 16, 4, 64, 700
    cache = ops.KVCache(B, n_kv, D, 704)
    cache.write(n(B, S, n_kv, D, std=1.0), n(B, S, n_kv, D, std=1.0), 0)
    attn = ops.AttnDecode(B, n_q, n_kv, D, S)
    lens = torch.randint(1, S + 1, (B,), device=dev, generator=g, dtype=torch.int32)
    sinks = torch.randn(n_q, device=dev, generator=g)

    t = n(B, H, std=1.0)
    q = torch.randn(B, n_q, D, device=dev, generator=g)
    y = torch.empty(B, H, dtype=torch.float32, device=dev)
    o = torch.empty(B, n_q, D, dtype=torch.bfloat16, device=dev)

    # no warm-up call: the first launches of these kernels in the process are the captured ones
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        layer.forward(t, y)
        attn.forward(q, cache, lens, sinks, window=0, out=o)

    for it in range(4):
        t.copy_(n(B, H, std=1.0))
        q.copy_(torch.randn(B, n_q, D, device=dev, generator=g))
        graph.replay()
        torch.cuda.synchronize()
        y_graph, o_graph = y.clone(), o.clone()
        # eager work between the replays, on the same workspaces
        y_eager = layer.forward(t).clone()
        o_eager = attn.forward(q, cache, lens, sinks, window=0).clone()
        torch.cuda.synchronize()
        assert torch.equal(y_graph, y_eager), it
        assert torch.equal(o_graph, o_eager), it
        assert np.isfinite(y_graph.cpu().numpy()).all()
