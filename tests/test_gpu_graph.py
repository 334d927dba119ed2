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


def test_drop_in_blocks_under_graph_capture(dev):
    """Four drop-in blocks called the way the reference's decoder calls them (same token-type tensor and CPU row
    ranges for every layer) recorded into a HIP graph: the first block's partition is recorded, the others reuse it
    within the capture, and every replay equals the eager result on the same inputs.  What the blocks keep between
    calls (the cached partition, the shared work buffers) must not leak out of the capture, where nothing has executed
    yet: an eager call right after the capture, on the capture's inputs, is checked as well."""
    from types import SimpleNamespace

    g = torch.Generator(device=dev).manual_seed(21)
    hidden, inters, n_vl, n_act = 512, (768, 256), 300, 212
    T = n_vl + n_act
    cfg = SimpleNamespace(experts=[dict(hidden_size=hidden, intermediate_size=i, hidden_act="silu") for i in inters])
    blocks = []
    for _ in range(4):
        b = moe.SparseMoeBlock(cfg, 2).to(dev).to(torch.bfloat16)
        with torch.no_grad():
            for prm in b.parameters():
                prm.copy_((torch.randn(prm.shape, device=dev, generator=g) * 0.03).to(torch.bfloat16))
        blocks.append(b.pack_for_inference())
    x_static = torch.zeros(1, T, hidden, dtype=torch.bfloat16, device=dev)
    types_static = torch.zeros(1, T, dtype=torch.bool, device=dev)
    start, end = torch.tensor([0, n_vl]), torch.tensor([n_vl, T])

    def run(x, types):
        h = x
        with torch.no_grad():
            for b in blocks:
                h = b(h, types, start, end, residual=True)
        return h

    def fill(it):
        gi = torch.Generator(device=dev).manual_seed(100 + it)
        x = torch.randn(1, T, hidden, device=dev, generator=gi).to(torch.bfloat16)
        types = torch.zeros(T, dtype=torch.bool, device=dev)
        types[torch.randperm(T, device=dev, generator=gi)[:n_act]] = True
        return x, types.view(1, T)

    x0, t0 = fill(0)
    x_static.copy_(x0)
    types_static.copy_(t0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(x_static, types_static)  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    want0 = run(x0, t0)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        out_static = run(x_static, types_static)
    # nothing of the capture has executed: an eager call on the same tensor objects AND the capture's stream must
    # partition for itself
    with torch.cuda.stream(side):
        eager_after = run(x_static, types_static)
    side.synchronize()
    assert torch.equal(eager_after, want0), "an eager call after the capture used state recorded inside it"
    torch.cuda.current_stream().wait_stream(side)

    for it in range(1, 4):
        x, types = fill(it)
        x_static.copy_(x)
        types_static.copy_(types)
        graph.replay()
        got = out_static.clone()
        torch.cuda.synchronize()
        want = run(x, types)  # eager work between the replays, on the same inputs
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {it} differs from the eager run"


def test_prefill_forward_graph_replays_match_eager(dev):
    """The whole harness forward (position builder, partition, per-layer projections / M-RoPE / attention on
    PyTorch-ROCm, fused movers and both FFN launches) recorded once and replayed on fresh inputs: every replay equals
    the eager forward on the same inputs, with eager work and synchronisations between the replays."""
    from wallx_mi355 import harness, workloads as wl

    h = harness.PrefillHarness(n_layers=2, hidden=256, n_q=4, n_kv=2, head_dim=128, inter=(512, 256), vocab=151936,
                               device=dev, seed=5)
    row = wl.vla_row_tokens(n_images=1, image_tokens=16, lead_text=5, tail_text=9, n_action=8)
    ids_static = torch.tensor([row, row], dtype=torch.int64, device=dev)
    grid = torch.tensor([[1, 8, 8]] * 2, dtype=torch.int64, device=dev)
    types_static = ids_static == wl.ACTION_TOKEN_ID

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        h.forward(ids_static, grid, types_static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static = h.forward(ids_static, grid, types_static)

    g = torch.Generator().manual_seed(0)
    for it in range(3):
        # same layout, other text tokens: the embedding rows (hence every activation) change
        ids = ids_static.clone().cpu()
        is_text = ids == wl.TEXT_TOKEN_ID
        ids[is_text] = torch.randint(1000, 2000, (int(is_text.sum()),), generator=g)
        ids = ids.to(dev)
        ids_static.copy_(ids)
        graph.replay()
        got = out_static.clone()
        torch.cuda.synchronize()
        want = h.forward(ids, grid, ids == wl.ACTION_TOKEN_ID)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"replay {it} differs from the eager forward"


def test_row_counts_reach_the_host_without_a_sync_and_captures_ignore_them(dev):
    """An eager partition starts an asynchronous copy of expert_offsets to pinned host memory; once it has landed,
    later layers hand the row counts to the GEMM entry points (one dispatch each instead of one per tile shape).  The
    result is the same either way, a partition made under capture has no such copy, and a capture that uses an eager
    routing still records the launches that decide on the device (its replays follow new offsets)."""
    g = torch.Generator(device=dev).manual_seed(23)
    hidden, inters = 1024, (1536, 512)
    weights = _weights(dev, hidden, inters, g)
    T, n_act = 2048, 2048
    x = torch.randn(T, hidden, device=dev, generator=g).to(torch.bfloat16)
    types = torch.ones(T, dtype=torch.bool, device=dev)
    routing = moe._routing_cache.lookup(types, 2)  # what a block's forward does with its token types
    assert routing.host_rows is not None
    y_first, _ = moe.moe_layer_forward(x, types, weights, routing=routing)  # most likely too early for the counts
    torch.cuda.synchronize()
    rows = routing.rows_when_ready()
    assert rows is not None and list(rows) == [T - n_act, n_act]
    y_host, _ = moe.moe_layer_forward(x, types, weights, routing=routing)  # now with the counts from the host
    assert int((y_first != y_host).sum()) == 0

    # a capture on an eager routing: the offsets change before the replay, and the replay follows them
    types_static = types.clone()
    x_static = x.clone()
    rmap, off, inv, _ = native.partition(types_static, 2, 0, None, want_sorted=True)
    static_routing = moe.Routing(rmap, off, T, inv)
    static_routing.host_rows = native.HostRows(off, T)
    for e in weights:
        for w in e:
            native.pack_weight(w)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        moe.moe_layer_forward(x_static, types_static, weights, routing=static_routing)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert static_routing.rows_when_ready() is not None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_static, _ = moe.moe_layer_forward(x_static, types_static, weights, routing=static_routing)
        captured, _ = moe.moe_layer_forward(x_static, types_static, weights)
        in_capture = moe._routing_cache.lookup(types_static, 2)
    assert in_capture.host_rows is None  # partitioned under capture: nothing has run, nothing to read back
    for n_vl in (0, 700):
        new_types = torch.ones(T, dtype=torch.bool, device=dev)
        new_types[:n_vl] = False
        types_static.copy_(new_types)
        # the eager routing's tensors are rewritten in place by a new partition, as a caller with static buffers would
        r2, o2, i2, _ws = native.partition(types_static, 2, 0, None, want_sorted=True)
        rmap.copy_(r2); off.copy_(o2); inv.copy_(i2)
        graph.replay()
        got, got_captured = out_static.clone(), captured.clone()
        torch.cuda.synchronize()
        want, _r = moe.moe_layer_forward(x, new_types, weights)
        torch.cuda.synchronize()
        assert int((got != want).sum()) == 0 and int((got_captured != want).sum()) == 0
