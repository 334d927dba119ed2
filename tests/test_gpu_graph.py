"""The layer's launches recorded once into a HIP graph and replayed: the denoise loop of config 4 runs the same
2048-token layer shape 10 x 36 times per action chunk, and at 5 launches of a few microseconds each it is bound by
launch overhead.  Every entry point enqueues on the caller's stream and neither allocates nor synchronises, so the
layer is capturable as it stands.  Each replay is checked against the eager result on the same inputs, with eager
work and synchronisations between the replays."""

import pytest
import torch

from wallx_mi355 import moe, native

pytestmark = pytest.mark.gpu


def _weights(dev, hidden, inters, g):
    out = []
    for inter in inters:
        mk = lambda *s: (torch.randn(*s, device=dev, generator=g) * 0.02).to(torch.bfloat16)
        out.append((mk(inter, hidden), mk(inter, hidden), mk(hidden, inter)))
    return out


@pytest.mark.parametrize("n_vl,n_act", [(0, 2048), (600, 40)])
def test_layer_graph_replays_match_eager(dev, n_vl, n_act):
    g = torch.Generator(device=dev).manual_seed(11)
    hidden, inters = 2048, (1024 + 256, 1024)
    weights = _weights(dev, hidden, inters, g)
    for e in weights:  # packing allocates and caches per weight; do it outside the capture
        for w in e:
            native.pack_weight(w)
    T = n_vl + n_act
    x_static = torch.zeros(T, hidden, dtype=torch.bfloat16, device=dev)
    types_static = torch.zeros(T, dtype=torch.bool, device=dev)
    layers = 3

    def run():
        h, routing = x_static, None
        for _ in range(layers):  # routing is shared by every layer of a forward, like the reference's caller does
            y, routing = moe.moe_layer_forward(h, types_static, weights, routing=routing)
            h = h + y
        return h

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()  # warm-up outside the capture (lazy initialisation, workspace sizes)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static = run()

    for it in range(4):
        x = torch.randn(T, hidden, device=dev, generator=g).to(torch.bfloat16)
        perm = torch.randperm(T, device=dev, generator=g)
        types = torch.zeros(T, dtype=torch.bool, device=dev)
        types[perm[:n_act]] = True  # same split, different token order on every replay
        x_static.copy_(x)
        types_static.copy_(types)
        graph.replay()
        got = out_static.clone()
        torch.cuda.synchronize()
        # eager work of the program between replays, on the same inputs
        h, routing = x, None
        for _ in range(layers):
            y, routing = moe.moe_layer_forward(h, types, weights, routing=routing)
            h = h + y
        torch.cuda.synchronize()
        assert routing.expert_offsets.cpu().tolist() == [0, n_vl, T]
        assert int((got != h).sum()) == 0, f"replay {it} differs from the eager run"
