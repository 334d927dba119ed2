"""The two GEMM launches of the dual-expert FFN as one launch (wx_dual_swiglu_ffn_fused: gate/up tiles and down tiles in
one grid, a down tile waiting on counters for the gate/up tiles of its rows) against the two launches it replaces
(act.py:79-82, 142-154 per expert): bit-equal results, a workspace that every call leaves zero, the shapes it hands
back to the two launches, and HIP graph replays."""

import pytest
import torch

import oracle
from wallx_mi355 import _lib, native

pytestmark = pytest.mark.gpu


def _case(dev, T, m0, H, I0, I1, seed):
    g = torch.Generator().manual_seed(seed)
    ws = [(torch.randn(s, generator=g) * 0.03).to(torch.bfloat16).to(dev)
          for s in ((I0, H), (I0, H), (H, I0), (I1, H), (I1, H), (H, I1))]
    packed = [native.pack_weight(w, cache=False) for w in ws]
    types = torch.cat([torch.zeros(m0, dtype=torch.bool), torch.ones(T - m0, dtype=torch.bool)])
    types = types[torch.randperm(T, generator=g)].to(dev)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    res = torch.randn(T, H, generator=g).to(torch.bfloat16).to(dev)
    rmap, off, inv, _ = native.partition(types, 2, 0, None, want_sorted=True)
    xt = native.permute_rows_tiled(x, rmap, off, None, inv)
    return ws, packed, types, x, res, off, inv, xt


def _workspace(dev):
    return torch.zeros(_lib.load().wx_ffn_fused_workspace_bytes() // 4, dtype=torch.int32, device=dev)


def _two_launches(p, xt, hm, out, res, off, inv, T, H, I0, I1, rows, stream):
    _lib.call("wx_dual_swiglu_gate_up", xt.data_ptr(), hm.data_ptr(), off.data_ptr(), p[0], p[1], p[3], p[4], T, H, I0, I1,
              rows, stream)
    if res is not None:
        _lib.call("wx_dual_down_proj_residual", hm.data_ptr(), out.data_ptr(), res.data_ptr(), off.data_ptr(), p[2], p[5],
                  T, H, I0, I1, rows, inv.data_ptr(), stream)
    else:
        _lib.call("wx_dual_down_proj", hm.data_ptr(), out.data_ptr(), off.data_ptr(), p[2], p[5], T, H, I0, I1, rows,
                  inv.data_ptr(), stream)


def _one_launch(p, xt, hm, out, res, off, inv, T, H, I0, I1, rows, ws, stream, x_rows=None):
    """x_rows: the activations in token order; xt is then the buffer that the call permutes them into."""
    _lib.call("wx_dual_swiglu_ffn_fused", None if x_rows is None else x_rows.data_ptr(), xt.data_ptr(), out.data_ptr(),
              None if res is None else res.data_ptr(), off.data_ptr(), p[0], p[1], p[2], p[3], p[4], p[5], hm.data_ptr(),
              T, H, I0, I1, rows, inv.data_ptr(), None if ws is None else ws.data_ptr(), stream)


# one round of 128 x 128 tiles per GEMM (the shapes that run as one launch): a denoise step's 2048 action tokens, all
# rows on expert 0, both experts with ragged tiles, a single row on one expert; then shapes that go to two launches
@pytest.mark.parametrize("T,m0,H,I0,I1,with_res,known_rows", [
    (2048, 0, 2048, 1536, 1024, False, True), (2048, 0, 2048, 1536, 1024, True, True), (1024, 1024, 256, 512, 1024, False, True),
    (1500, 700, 512, 448, 320, True, True), (129, 1, 1024, 64, 1024, False, True), (300, 300, 96, 32, 32, True, True),
    (2048, 0, 2048, 1536, 1024, False, False),   # rows only known on the device: too many for the one launch ...
    (512, 0, 2048, 1536, 1024, False, False), (300, 200, 512, 448, 320, True, False),   # ... and few enough for it
    (4096, 100, 2048, 1024, 1024, True, True),   # more tiles than CUs
])
def test_one_launch_ffn_equals_two_launches(dev, T, m0, H, I0, I1, with_res, known_rows):
    ws_, packed, types, x, res, off, inv, xt = _case(dev, T, m0, H, I0, I1, T + H + I0)
    p = [t.data_ptr() for t in packed]
    stream = torch.cuda.current_stream().cuda_stream
    pad = native.padded_sorted_rows(T)
    hm = [torch.zeros(pad * max(I0, I1), dtype=torch.bfloat16, device=dev) for _ in range(2)]
    out = [torch.full((T, H), v, dtype=torch.bfloat16, device=dev) for v in (7.0, 9.0)]
    rows = _lib.i64x2((m0, T - m0)) if known_rows else None
    r = res if with_res else None
    work = _workspace(dev)
    _two_launches(p, xt, hm[0], out[0], r, off, inv, T, H, I0, I1, rows, stream)
    xt2 = torch.full_like(xt, 3.0)
    for call in range(4):  # every call after the first runs on the workspace the one before it left
        out[1].fill_(9.0)
        if call < 2:
            _one_launch(p, xt, hm[1], out[1], r, off, inv, T, H, I0, I1, rows, work, stream)
        else:  # ... and with the permute inside the launch (the gate/up tiles read the token rows)
            _one_launch(p, xt2, hm[1], out[1], r, off, inv, T, H, I0, I1, rows, work, stream, x_rows=x)
        torch.cuda.synchronize()
        assert torch.equal(out[0], out[1]), f"call {call}"
        assert torch.equal(hm[0], hm[1]), f"call {call}"
        assert int(work.abs().sum()) == 0, f"call {call}: counters or the error flag left set"
    # against the oracle
    wc = [tuple(w.cpu() for w in ws_[:3]), tuple(w.cpu() for w in ws_[3:])]
    ref = oracle.sparse_moe_block_ref(x.cpu()[None], types.cpu()[None], wc)[0].float()
    if with_res:
        ref = (res.cpu().float() + ref).to(torch.bfloat16).float()
    err = (out[1].cpu().float() - ref).abs()
    assert not (err > 2e-2 + 1e-2 * ref.abs()).any(), float(err.max())


@pytest.mark.parametrize("hint", [(4096, 0), (3968, 128), (128, 3968), (0, 4096)])
def test_one_launch_ffn_with_row_counts_that_are_not_the_devices(dev, hint):
    """The host's row counts choose the launch; the kernels read the split from expert_offsets.  Counts that are not
    the device's (here 2049 + 2047 rows) may pick the one launch for a problem with more tiles than it has workgroups
    for -- gate/up workgroups then take several tiles each, and so do down workgroups, each tile behind its own wait
    -- and the result does not change."""
    T, m0, H, I0, I1 = 4096, 2049, 1024, 64, 1024
    _, packed, _, x, res, off, inv, xt = _case(dev, T, m0, H, I0, I1, 17)
    p = [t.data_ptr() for t in packed]
    stream = torch.cuda.current_stream().cuda_stream
    pad = native.padded_sorted_rows(T)
    hm = [torch.zeros(pad * max(I0, I1), dtype=torch.bfloat16, device=dev) for _ in range(2)]
    out = [torch.full((T, H), v, dtype=torch.bfloat16, device=dev) for v in (7.0, 9.0)]
    work = _workspace(dev)
    _two_launches(p, xt, hm[0], out[0], res, off, inv, T, H, I0, I1, None, stream)
    xt2 = torch.full_like(xt, 3.0)
    for call in range(2):
        if call == 0:
            _one_launch(p, xt, hm[1], out[1], res, off, inv, T, H, I0, I1, _lib.i64x2(hint), work, stream)
        else:
            _one_launch(p, xt2, hm[1], out[1], res, off, inv, T, H, I0, I1, _lib.i64x2(hint), work, stream, x_rows=x)
        torch.cuda.synchronize()
        assert torch.equal(out[0], out[1]) and torch.equal(hm[0], hm[1]), f"call {call}"
        assert int(work.abs().sum()) == 0


def test_one_launch_ffn_without_a_workspace_is_the_two_launches(dev):
    T, m0, H, I0, I1 = 700, 200, 256, 384, 128
    _, packed, _, _, _, off, inv, xt = _case(dev, T, m0, H, I0, I1, 5)
    p = [t.data_ptr() for t in packed]
    stream = torch.cuda.current_stream().cuda_stream
    pad = native.padded_sorted_rows(T)
    hm = [torch.zeros(pad * max(I0, I1), dtype=torch.bfloat16, device=dev) for _ in range(2)]
    out = [torch.empty(T, H, dtype=torch.bfloat16, device=dev) for _ in range(2)]
    rows = _lib.i64x2((m0, T - m0))
    _two_launches(p, xt, hm[0], out[0], None, off, inv, T, H, I0, I1, rows, stream)
    _one_launch(p, xt, hm[1], out[1], None, off, inv, T, H, I0, I1, rows, None, stream)
    torch.cuda.synchronize()
    assert torch.equal(out[0], out[1]) and torch.equal(hm[0], hm[1])
    lib = _lib.load()
    work = _workspace(dev)
    assert lib.wx_dual_swiglu_ffn_fused(None, xt.data_ptr(), out[1].data_ptr(), None, off.data_ptr(), *p, hm[1].data_ptr(),
                                        T, H, I0, I1, rows, inv.data_ptr(), work.data_ptr() + 2, stream) == -1
    assert b"aligned" in lib.wx_last_error_string()
    assert lib.wx_dual_swiglu_ffn_fused(None, xt.data_ptr(), out[1].data_ptr(), out[0].data_ptr(), off.data_ptr(), *p,
                                        hm[1].data_ptr(), T, H, I0, I1, rows, None, work.data_ptr(), stream) == -1
    assert b"out_row_id" in lib.wx_last_error_string()  # a residual is added in token order
    assert lib.wx_dual_swiglu_ffn_fused(out[0].data_ptr(), xt.data_ptr(), out[1].data_ptr(), None, off.data_ptr(), *p,
                                        hm[1].data_ptr(), T, H, I0, I1, rows, None, work.data_ptr(), stream) == -1
    assert b"out_row_id" in lib.wx_last_error_string()  # ... and rows are gathered through it


def test_one_launch_ffn_replays_from_a_hip_graph(dev):
    """Captured once, replayed with the program's own eager launches and synchronisations in between: every replay
    equals the eager result, and the counters are zero after each."""
    T, m0, H, I0, I1 = 2048, 0, 1024, 512, 1024
    _, packed, _, x, res, off, inv, xt = _case(dev, T, m0, H, I0, I1, 11)
    p = [t.data_ptr() for t in packed]
    pad = native.padded_sorted_rows(T)
    rows = _lib.i64x2((m0, T - m0))
    hm = [torch.zeros(pad * max(I0, I1), dtype=torch.bfloat16, device=dev) for _ in range(2)]
    out = [torch.empty(T, H, dtype=torch.bfloat16, device=dev) for _ in range(2)]
    work = _workspace(dev)
    _two_launches(p, xt, hm[0], out[0], res, off, inv, T, H, I0, I1, rows, torch.cuda.current_stream().cuda_stream)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        _one_launch(p, xt, hm[1], out[1], res, off, inv, T, H, I0, I1, rows, work, side.cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    xt2 = torch.zeros_like(xt)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _one_launch(p, xt2, hm[1], out[1], res, off, inv, T, H, I0, I1, rows, work,
                    torch.cuda.current_stream().cuda_stream, x_rows=x)
    for replay in range(4):
        out[1].zero_()
        hm[1].zero_()
        xt2.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out[0], out[1]) and torch.equal(hm[0], hm[1]), f"replay {replay}"
        assert int(work.abs().sum()) == 0
        # eager work of the program between replays, on the same workspace
        _one_launch(p, xt, hm[1], out[1], res, off, inv, T, H, I0, I1, rows, work, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert torch.equal(out[0], out[1])


@pytest.mark.parametrize("residual", [False, True])
def test_block_forward_with_and_without_the_one_launch_ffn(dev, residual, monkeypatch):
    """native.packed_block_forward (wx_moe_block_forward) hands the library its per-stream counter workspace; switched
    off, it makes the two launches.  Same bits."""
    T, H, I0, I1 = 1024, 512, 768, 256
    g = torch.Generator().manual_seed(3)
    ws = [(torch.randn(s, generator=g) * 0.05).to(torch.bfloat16).to(dev)
          for s in ((I0, H), (I0, H), (H, I0), (I1, H), (I1, H), (H, I1))]
    experts = native.PackedExperts([native.pack_weight(w, cache=False) for w in ws], (H, I0, I1))
    types = (torch.rand(T, generator=g) < 0.3).to(dev)
    x = (torch.randn(T, H, generator=g) * 2.0).to(torch.bfloat16).to(dev)
    rmap, off, inv, _ = native.partition(types, 2, 0, None, want_sorted=True)
    n1 = int(types.sum())
    rows = _lib.i64x2((T - n1, n1))
    got = {}
    for flag in (True, False):
        monkeypatch.setattr(native, "_one_launch_ffn", flag)  # (what native.set_one_launch_ffn sets)
        got[flag] = native.packed_block_forward(experts, x, rmap, inv, off, rows, residual=residual)
    torch.cuda.synchronize()
    assert torch.equal(got[True], got[False])


def test_one_launch_ffn_on_two_streams_at_once(dev):
    """Two streams issue the one launch at the same time, each with a workspace of its own (what
    native.packed_block_forward keeps per stream): workgroups of both launches share the CUs, each launch's down tiles
    wait on its own counters, and both results are those of the separate launches.  (With two such launches resident
    an XCD's 64 workgroup places cannot all be held by waiting down workgroups of the other launch -- one launch has
    at most 32 of them per XCD -- so the gate/up workgroups of either always find a place.)"""
    T, m0, H, I0, I1 = 2048, 0, 2048, 1536, 1024
    pad = native.padded_sorted_rows(T)
    rows = _lib.i64x2((m0, T - m0))
    lanes = []
    for seed in (21, 22):
        _, packed, _, x, res, off, inv, xt = _case(dev, T, m0, H, I0, I1, seed)
        p = [t.data_ptr() for t in packed]
        hm = [torch.zeros(pad * max(I0, I1), dtype=torch.bfloat16, device=dev) for _ in range(2)]
        out = [torch.empty(T, H, dtype=torch.bfloat16, device=dev) for _ in range(2)]
        _two_launches(p, xt, hm[0], out[0], res, off, inv, T, H, I0, I1, rows, torch.cuda.current_stream().cuda_stream)
        lanes.append(dict(packed=packed, p=p, x=x, res=res, off=off, inv=inv, xt=torch.zeros_like(xt), hm=hm, out=out,
                          work=_workspace(dev), stream=torch.cuda.Stream()))
    torch.cuda.synchronize()
    for rep in range(3):
        for ln in lanes:
            ln["out"][1].zero_()
            ln["hm"][1].zero_()
        torch.cuda.synchronize()
        for _ in range(12):  # the host issues faster than a launch runs: the two streams' launches overlap
            for ln in lanes:
                _one_launch(ln["p"], ln["xt"], ln["hm"][1], ln["out"][1], ln["res"], ln["off"], ln["inv"], T, H, I0, I1,
                            rows, ln["work"], ln["stream"].cuda_stream, x_rows=ln["x"])
        torch.cuda.synchronize()
        for i, ln in enumerate(lanes):
            assert torch.equal(ln["out"][0], ln["out"][1]) and torch.equal(ln["hm"][0], ln["hm"][1]), f"rep {rep} stream {i}"
            assert int(ln["work"].abs().sum()) == 0, f"rep {rep} stream {i}: counters or the error flag left set"
