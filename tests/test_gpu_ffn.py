"""GPU parity: dual asymmetric grouped GEMM, fused dual-expert SwiGLU FFN and the MoE block.
Tolerance for bf16 outputs (fp32 accumulate): |x - ref| <= 2e-2 + 1e-2 |ref|."""

import pytest
import torch

import oracle
from wallx_mi355 import moe, native, workloads as wl
from wallx_mi355.fusions import ops

pytestmark = pytest.mark.gpu

ATOL, RTOL = 2e-2, 1e-2


def _close(got, ref, atol=ATOL, rtol=RTOL, what=""):
    got, ref = got.float().cpu(), ref.float().cpu()
    assert got.shape == ref.shape
    err = (got - ref).abs()
    bad = err > atol + rtol * ref.abs()
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance, max abs err {float(err.max())}"


def _bf(shape, g, std=1.0):
    return (torch.randn(shape, generator=g) * std).to(torch.bfloat16)


GEMM_SHAPES = [
    # m0, n0, k0, m1, n1, k1
    (256, 256, 64, 256, 256, 64),        # exactly one tile each
    (300, 264, 128, 40, 72, 192),        # ragged M and N
    (1, 8, 8, 1, 8, 8),                  # minimum
    (513, 1024, 2048, 31, 128, 2048),    # skewed pair
    (0, 256, 64, 77, 520, 72),           # empty VL group, K not a multiple of 64
    (129, 136, 200, 0, 64, 64),          # empty action group, K tail
    (0, 64, 64, 0, 64, 64),              # nothing to do
    (3000, 3080, 96, 200, 264, 160),     # enough 256 x 256 tiles to take the large-tile kernel, ragged everywhere
    (40, 64, 0, 24, 72, 64),             # empty contraction: the output is zeros
]


@pytest.mark.parametrize("shape", GEMM_SHAPES)
@pytest.mark.parametrize("trans_b", [True, False])
def test_dual_gemm(dev, shape, trans_b):
    m0, n0, k0, m1, n1, k1 = shape
    g = torch.Generator().manual_seed(sum(shape))
    a0, a1 = _bf((m0, k0), g), _bf((m1, k1), g)
    w0 = _bf((n0, k0) if trans_b else (k0, n0), g, 0.05)
    w1 = _bf((n1, k1) if trans_b else (k1, n1), g, 0.05)
    r0, r1 = oracle.dual_gemm_ref(a0, a1, w0, w1, False, trans_b)
    o0, o1 = ops.asym_dual_gmm(a0.to(dev), a1.to(dev), w0.to(dev), w1.to(dev), trans_b=trans_b)
    assert o0.dtype == torch.bfloat16 and o0.shape == (m0, n0) and o1.shape == (m1, n1)
    _close(o0, r0, what="expert 0")
    _close(o1, r1, what="expert 1")


def test_dual_gemm_mfma_path_is_tight(dev):
    """fp32 accumulation + one bf16 rounding: the error against a float64 contraction stays within half a bf16
    ulp plus accumulation noise, far inside the stated tolerance (catches a dropped K slab or a swapped fragment)."""
    g = torch.Generator().manual_seed(0)
    a0, a1 = _bf((512, 1024), g), _bf((96, 512), g)
    w0, w1 = _bf((768, 1024), g, 0.03), _bf((320, 512), g, 0.03)
    o0, o1 = ops.asym_dual_gmm(a0.to(dev), a1.to(dev), w0.to(dev), w1.to(dev), trans_b=True)
    for o, a, w in ((o0, a0, w0), (o1, a1, w1)):
        exact = a.double() @ w.double().T
        assert torch.all((o.cpu().double() - exact).abs() <= exact.abs() * 2 ** -8 + 2e-3)


def test_dual_gemm_all_transposes_and_autograd(dev):
    g = torch.Generator().manual_seed(3)
    a0, a1 = _bf((72, 64), g), _bf((40, 128), g)
    w0, w1 = _bf((96, 64), g, 0.1), _bf((56, 128), g, 0.1)
    for ta in (False, True):
        for tb in (False, True):
            x0, x1 = (a0.t().contiguous(), a1.t().contiguous()) if ta else (a0, a1)
            v0, v1 = (w0, w1) if tb else (w0.t().contiguous(), w1.t().contiguous())
            o0 = torch.empty(72, 96, dtype=torch.bfloat16, device=dev)
            o1 = torch.empty(40, 56, dtype=torch.bfloat16, device=dev)
            native.asym_dual_gmm(x0.to(dev), x1.to(dev), v0.to(dev), v1.to(dev), o0, o1, ta, tb)
            r0, r1 = oracle.dual_gemm_ref(x0, x1, v0, v1, ta, tb)
            _close(o0, r0, what=f"ta={ta} tb={tb}")
            _close(o1, r1, what=f"ta={ta} tb={tb}")
    # autograd contract of ops.py:78-144 against torch autograd on the fp32 restatement
    for tb in (True, False):
        v0, v1 = (w0, w1) if tb else (w0.t().contiguous(), w1.t().contiguous())
        leaves = [t.to(dev).requires_grad_(True) for t in (a0, a1, v0, v1)]
        o0, o1 = ops.asym_dual_gmm(*leaves, trans_b=tb)
        g0, g1 = _bf(o0.shape, g), _bf(o1.shape, g)
        torch.autograd.backward([o0, o1], [g0.to(dev), g1.to(dev)])
        refs = [t.float().requires_grad_(True) for t in (a0, a1, v0, v1)]
        p0 = refs[0] @ (refs[2].t() if tb else refs[2])
        p1 = refs[1] @ (refs[3].t() if tb else refs[3])
        torch.autograd.backward([p0, p1], [g0.float(), g1.float()])
        for leaf, ref in zip(leaves, refs):
            _close(leaf.grad, ref.grad, atol=6e-2, rtol=1e-2, what=f"grad trans_b={tb}")


@pytest.mark.parametrize("shape", [(8, 8), (64, 64), (200, 72), (1000, 136), (24, 4096)])
def test_transpose_2d_is_exact(dev, shape):
    g = torch.Generator().manual_seed(shape[0])
    t = _bf(shape, g).to(dev)
    assert torch.equal(native.transpose_2d(t), t.t().contiguous())


@pytest.mark.parametrize("shape", [
    # m0, n0, k0, m1, n1, k1
    (72, 96, 64, 40, 56, 128),            # small tiles
    (3000, 3080, 96, 200, 264, 160),      # large tiles, ragged everywhere
    (264, 520, 2048, 0, 64, 64),          # long contraction, empty second problem
])
def test_dual_gemm_k_major_layouts_through_the_c_abi(dev, shape):
    """Operands stored with K as the slow dimension (A as [k, m], B as [k, n]: the layouts of the backward GEMMs,
    ops.py:78-144) are read in place and transposed between LDS and the registers; straight through the C ABI."""
    from wallx_mi355 import _lib

    m0, n0, k0, m1, n1, k1 = shape
    g = torch.Generator().manual_seed(5)
    for ta, tb in ((False, False), (True, False), (True, True)):
        kk0, kk1 = (k0 + 13, k1 + 3) if (ta and not tb) else (k0, k1)  # K rows need no alignment when both are K-major
        a0, a1 = _bf((m0 // 8 * 8 if ta else m0, kk0), g), _bf((m1 // 8 * 8 if ta else m1, kk1), g)
        w0, w1 = _bf((n0, kk0), g, 0.1), _bf((n1, kk1), g, 0.1)
        x0, x1 = (a0.t().contiguous(), a1.t().contiguous()) if ta else (a0, a1)
        v0, v1 = (w0, w1) if tb else (w0.t().contiguous(), w1.t().contiguous())
        d = [t.to(dev) for t in (x0, x1, v0, v1)]
        o0 = torch.full((a0.size(0), n0), 7.0, dtype=torch.bfloat16, device=dev)
        o1 = torch.full((a1.size(0), n1), 7.0, dtype=torch.bfloat16, device=dev)
        _lib.call("wx_dual_gemm", d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(), o0.data_ptr(),
                  o1.data_ptr(), a0.size(0), n0, kk0, a1.size(0), n1, kk1, int(ta), int(tb),
                  torch.cuda.current_stream().cuda_stream)
        r0, r1 = oracle.dual_gemm_ref(x0, x1, v0, v1, ta, tb)
        _close(o0, r0, what=f"C ABI ta={ta} tb={tb}")
        _close(o1, r1, what=f"C ABI ta={ta} tb={tb}")


def test_dual_gemm_rejects_what_the_reference_rejects(dev):
    a = torch.zeros(8, 8, device=dev)
    with pytest.raises(RuntimeError, match="BFloat16"):
        ops.asym_dual_gmm(a, a, a, a)
    b = torch.zeros(8, 8, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="CUDA"):
        ops.asym_dual_gmm(b, b, b, b)


def _moe_weights(hidden, inters, g, std=0.02):
    return [wl.expert_weights(hidden, i, torch.bfloat16, g, std) for i in inters]


@pytest.mark.parametrize("T,n_act,hidden,inters", [
    (512, 64, 256, (384, 128)),
    (700, 33, 512, (1056, 160)),
    (300, 0, 256, (256, 128)),
    (300, 300, 256, (256, 128)),
    (1, 1, 64, (64, 64)),
])
def test_fused_ffn_small(dev, T, n_act, hidden, inters):
    g = torch.Generator().manual_seed(T + n_act)
    x = _bf((T, hidden), g)
    types = torch.zeros(T, dtype=torch.bool)
    types[torch.randperm(T, generator=g)[:n_act]] = True
    ws = _moe_weights(hidden, inters, g, 0.05)
    ref = oracle.sparse_moe_block_ref(x[None], types[None], [w.as_tuple() for w in ws])[0]
    y, routing = moe.moe_layer_forward(x.to(dev), types.to(dev), [w.to(dev).as_tuple() for w in ws])
    assert routing.expert_offsets.cpu().tolist() == [0, T - n_act, T]
    _close(y, ref, what="moe layer")
    ref32 = oracle.sparse_moe_block_ref(x[None], types[None], [w.as_tuple() for w in ws], eager_rounding=False)[0]
    # sanity bound against un-rounded fp32 math: eager rounding of the intermediates moves results a little
    _close(y, ref32, atol=2 * ATOL, rtol=2 * RTOL, what="moe layer vs fp32 math")


@pytest.mark.parametrize("T,n_act,hidden,inters", [
    (8600, 300, 2048, (1056, 256)),   # gate/up: 301 large tiles, 45 left over, among them a ragged last column
    (8600, 8300, 2048, (256, 1056)),  # the action expert is the long one
    (8600, 300, 2176, (512, 128)),    # down: 315 large tiles with a ragged last column; the short expert rides along
])
def test_fused_ffn_ragged_last_round(dev, T, n_act, hidden, inters):
    """More 256 x 256 tiles than CUs with a few left over: the whole rounds run as large tiles and the leftover as
    tiles of half the width in a second launch.  Whole output against the oracle, with the row split known only on
    the device and with it handed over from the host (right and wrong)."""
    g = torch.Generator().manual_seed(T + n_act + hidden)
    x = _bf((T, hidden), g)
    types = torch.zeros(T, dtype=torch.bool)
    types[torch.randperm(T, generator=g)[:n_act]] = True
    ws = _moe_weights(hidden, inters, g, 0.03)
    ref = oracle.sparse_moe_block_ref(x[None], types[None], [w.as_tuple() for w in ws])[0]
    wd = [w.to(dev).as_tuple() for w in ws]
    y, routing = moe.moe_layer_forward(x.to(dev), types.to(dev), wd)
    assert routing.expert_offsets.cpu().tolist() == [0, T - n_act, T]
    _close(y, ref, what="device-side split")
    for hint in ((T - n_act, n_act), (n_act, T - n_act), (T, 0)):
        yh, _ = moe.moe_layer_forward(x.to(dev), types.to(dev), wd, routing=routing, host_rows=hint)
        assert int((yh != y).sum()) == 0, f"host row counts {hint} changed the result"


@pytest.mark.parametrize("T,n_act,hidden,inters", [
    (700, 33, 512, (1056, 160)),      # small tiles
    (5000, 300, 2048, (512, 256)),    # large tiles, ragged rows
    (8600, 300, 2176, (512, 128)),    # large tiles + a ragged last round on the small-tile kernel, ragged columns
    (300, 300, 256, (256, 128)),      # one expert empty
])
def test_down_launch_stores_rows_at_their_token_positions(dev, T, n_act, hidden, inters):
    """wx_dual_swiglu_ffn with out_row_id (the partition's inverse map): the result in token order must equal the
    sorted-order result put through the stand-alone unpermute, bit for bit."""
    g = torch.Generator(device=dev).manual_seed(T + hidden)
    x = torch.randn(T, hidden, device=dev, generator=g).to(torch.bfloat16)
    types = torch.zeros(T, dtype=torch.bool, device=dev)
    types[torch.randperm(T, device=dev, generator=g)[:n_act]] = True
    ws = [w.to(dev).as_tuple() for w in _moe_weights(hidden, inters, torch.Generator().manual_seed(1), 0.03)]
    rmap, off, inv, _ = native.partition(types, 2, 0, None, want_sorted=True)
    x_tiled = native.permute_rows_tiled(x, rmap, off, None, inv)
    y_sorted = native.dual_swiglu_ffn(x_tiled, T, off, ws)
    want = native.unpermute(y_sorted, rmap, torch.tensor([]), T, 1)
    got = torch.full((T, hidden), float("nan"), dtype=torch.bfloat16, device=dev)
    native.dual_swiglu_ffn(x_tiled, T, off, ws, out=got, out_row_id=inv)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    for hint in ((T - n_act, n_act), (n_act, T - n_act)):
        got2 = native.dual_swiglu_ffn(x_tiled, T, off, ws, host_rows=hint, out_row_id=inv)
        assert torch.equal(got2.view(torch.int16), want.view(torch.int16))


def test_fused_ffn_intermediate_beyond_2_gib(dev):
    """131 072 tokens at the BASELINE widths: the VL expert's intermediate is 2.9 GB, past what a buffer descriptor's
    32-bit byte count holds, so the loads run with clamped counts.  Rows sampled across the whole range (first and
    last tiles of both experts included) against the oracle; every output finite."""
    T, n_act, H, inters = 131072, 4096, wl.HIDDEN, (wl.INTER_VL, wl.INTER_ACT)
    g = torch.Generator(device=dev).manual_seed(9)
    x = torch.randn(T, H, device=dev, generator=g).to(torch.bfloat16)
    types = torch.zeros(T, dtype=torch.bool, device=dev)
    types[torch.randperm(T, device=dev, generator=g)[:n_act]] = True
    gc = torch.Generator().manual_seed(9)
    ws = _moe_weights(H, inters, gc, 0.02)
    y, routing = moe.moe_layer_forward(x, types, [w.to(dev).as_tuple() for w in ws])
    assert routing.expert_offsets.cpu().tolist() == [0, T - n_act, T]
    assert bool(torch.isfinite(y.float()).all())
    inv = routing.sorted_row_id.long()
    picks = torch.cat([torch.arange(0, 8), torch.arange(T - n_act - 8, T - n_act + 8), torch.arange(T - 8, T),
                       torch.randint(0, T, (40,), generator=gc)]).to(dev)
    rows = inv[picks]  # tokens at chosen sorted positions
    ref = oracle.sparse_moe_block_ref(x[rows].cpu()[None], types[rows].cpu()[None], [w.as_tuple() for w in ws])[0]
    _close(y[rows], ref, what="sampled rows")


def test_moe_block_module_is_a_drop_in(dev):
    class Cfg:
        experts = [{"hidden_size": 256, "intermediate_size": 512, "hidden_act": "silu"},
                   {"hidden_size": 256, "intermediate_size": 128, "hidden_act": "silu"}]

    torch.manual_seed(0)
    block = moe.SparseMoeBlock(Cfg(), 2).to(torch.bfloat16)
    assert sorted(n for n, _ in block.named_parameters()) == sorted(
        f"experts.{e}.{p}_proj.weight" for e in (0, 1) for p in ("gate", "up", "down"))
    g = torch.Generator().manual_seed(1)
    x = _bf((2, 100, 256), g)
    types = torch.rand(2, 100, generator=g) > 0.8
    weights = [tuple(w.detach().clone() for w in e.weights()) for e in block.experts]
    ref = oracle.sparse_moe_block_ref(x, types, weights)
    block = block.to(dev)
    n0 = int((~types).sum())
    start, end = torch.tensor([0, n0]), torch.tensor([n0, 200])  # what the reference caller passes (act.py:1274-1283)
    with torch.no_grad():
        y = block(x.to(dev), types.to(dev), start, end)
        r = block.route(types.to(dev))
        y2 = block(x.to(dev), types.to(dev), routing=r)
    assert y.shape == (2, 100, 256)
    _close(y, ref, what="block")
    assert int((y != y2).sum()) == 0


def test_config1_golden_shapes_in_bf16(dev):
    """Config 1 (512 tokens, 448 VL + 64 action, fp32 golden on the CPU path).  The kernels are bf16, so the same
    seeded inputs are rounded to bf16 and compared with the fp32 golden within the stated tolerance."""
    x, types, ws = wl.config1()
    golden = oracle.sparse_moe_block_ref(x, types, [w.as_tuple() for w in ws])[0]  # fp32 throughout
    xb = x[0].to(torch.bfloat16)
    wb = [tuple(t.to(torch.bfloat16).to(dev) for t in w.as_tuple()) for w in ws]
    y, routing = moe.moe_layer_forward(xb.to(dev), types[0].to(dev), wb)
    assert routing.expert_offsets.cpu().tolist() == [0, 448, 512]
    assert torch.equal(routing.row_id_map.cpu(), torch.arange(512, dtype=torch.int32))
    # same bf16-rounded inputs through the oracle: the stated tolerance
    ref = oracle.sparse_moe_block_ref(xb[None], types, [tuple(t.to(torch.bfloat16) for t in w.as_tuple()) for w in ws])[0]
    _close(y, ref, what="config 1, bf16 inputs")
    # against the fp32 golden the rounding of the inputs and weights to bf16 adds its own error, so the bound is
    # wider: 4e-2 + 1e-2 |ref|, and the bulk of the outputs must sit inside the stated tolerance
    _close(y, golden, atol=4e-2, rtol=1e-2, what="config 1 vs fp32 golden")
    err = (y.float().cpu() - golden).abs()
    assert float((err <= ATOL + RTOL * golden.abs()).float().mean()) > 0.9999


def test_config3_rows_sample_at_full_size(dev):
    """Full config 3 (29184 x 2048, 28160 VL / 1024 action) on the GPU; the oracle is evaluated on a sample of
    token rows (each token's output depends only on its own row), covering both experts and tile edges."""
    x, types, ws = wl.config3()
    T = x.shape[0] * x.shape[1]
    xf, tf = x.view(T, -1), types.view(T)
    wd = [w.to(dev).as_tuple() for w in ws]
    y, routing = moe.moe_layer_forward(xf.to(dev), tf.to(dev), wd)
    assert routing.expert_offsets.cpu().tolist() == [0, 28160, 29184]
    g = torch.Generator().manual_seed(1)
    act_rows = torch.nonzero(tf).flatten()
    vl_rows = torch.nonzero(~tf).flatten()
    pick = torch.cat([vl_rows[torch.randperm(vl_rows.numel(), generator=g)[:96]], vl_rows[:4], vl_rows[-4:],
                      act_rows[torch.randperm(act_rows.numel(), generator=g)[:24]], act_rows[:2], act_rows[-2:]])
    ref = oracle.sparse_moe_block_ref(xf[pick][None], tf[pick][None], [w.as_tuple() for w in ws])[0]
    _close(y[pick.to(dev)], ref, what="config 3 sample")
    # linearity of the down projection in its weights is a size-independent property: doubling W_down doubles y
    wd2 = [(g_, u_, (2 * d_).contiguous()) for (g_, u_, d_) in wd]
    y2, _ = moe.moe_layer_forward(xf.to(dev), tf.to(dev), wd2, routing=routing)
    assert int((y2 != (2 * y.float()).to(torch.bfloat16)).sum()) == 0


def test_config4_skewed_and_empty_groups(dev):
    g = torch.Generator().manual_seed(4)
    ws = _moe_weights(2048, (1024 + 256, 1024), g, 0.02)  # a smaller VL expert keeps the CPU check quick
    wd = [w.to(dev).as_tuple() for w in ws]
    # (i) denoise step: 2048 action tokens, VL group empty
    x = _bf((2048, 2048), g)
    types = torch.ones(2048, dtype=torch.bool)
    y, r = moe.moe_layer_forward(x.to(dev), types.to(dev), wd)
    assert r.expert_offsets.cpu().tolist() == [0, 0, 2048]
    rows = torch.arange(0, 2048, 37)
    _close(y[rows.to(dev)], oracle.swiglu_ffn_ref(x[rows], *ws[1].as_tuple()), what="denoise step")
    # row counts handed over from the host only pick the tile shape: same result, right or wrong
    for hint in ((0, 2048), (2048, 0)):
        yh, _ = moe.moe_layer_forward(x.to(dev), types.to(dev), wd, host_rows=hint)
        assert int((yh != y).sum()) == 0
    # the same step next to a wide VL expert: the host cannot tell which tile shape fits (the row split is on the
    # device), so both are launched and the device picks
    ws_wide = _moe_weights(2048, (4096, 1024), g, 0.02)
    y2, _ = moe.moe_layer_forward(x.to(dev), types.to(dev), [w.to(dev).as_tuple() for w in ws_wide])
    _close(y2[rows.to(dev)], oracle.swiglu_ffn_ref(x[rows], *ws_wide[1].as_tuple()), what="denoise step, wide VL expert")
    # (ii) prefill: 4096 VL tokens + n action tokens, alternating with (i) without re-tuning
    for n_act in (0, 1, 8, 64):
        x = _bf((4096 + n_act, 2048), g)
        types = torch.cat([torch.zeros(4096, dtype=torch.bool), torch.ones(n_act, dtype=torch.bool)])
        y, r = moe.moe_layer_forward(x.to(dev), types.to(dev), wd)
        rows = torch.cat([torch.arange(0, 4096, 173), torch.arange(4096, 4096 + n_act)])
        ref = oracle.sparse_moe_block_ref(x[rows][None], types[rows][None], [w.as_tuple() for w in ws])[0]
        _close(y[rows.to(dev)], ref, what=f"prefill + {n_act} action")


@pytest.mark.parametrize("shape", [(1, 8), (37, 264), (300, 1056), (0, 64)])
def test_swiglu_bwd_kernel(dev, shape):
    g = torch.Generator().manual_seed(shape[0] + shape[1])
    gate, up, dh = _bf(shape, g, 2.0), _bf(shape, g), _bf(shape, g)
    hm, dg, du = native.swiglu_bwd(gate.to(dev), up.to(dev), dh.to(dev))
    rh, rg, ru = oracle.swiglu_bwd_ref(gate, up, dh)
    # fp32 math with the device's exp against the host's: a bf16 step where a result sits on a rounding boundary
    for got, ref, what in ((hm, rh, "hmid"), (dg, rg, "dgate"), (du, ru, "dup")):
        got, ref = got.float().cpu(), ref.float()
        bad = (got - ref).abs() > 2.0 ** -7 * ref.abs() + 1e-30
        assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} differ by more than a bf16 step"
        assert got.numel() == 0 or float((got != ref).float().mean()) < 0.02, what


@pytest.mark.parametrize("fused_extras", [False, True])
def test_moe_block_backward_matches_autograd_of_the_plain_forward(dev, fused_extras):
    """Gradients of the block (inputs and all six weights) against torch autograd through the oracle's fp32
    forward; with fused_extras the layer's RMSNorm and residual ride along (PyTorch ops under autograd)."""
    class Cfg:
        experts = [{"hidden_size": 128, "intermediate_size": 256, "hidden_act": "silu"},
                   {"hidden_size": 128, "intermediate_size": 64, "hidden_act": "silu"}]

    g = torch.Generator().manual_seed(12)
    block = moe.SparseMoeBlock(Cfg(), 2).to(torch.bfloat16)
    with torch.no_grad():
        for prm in block.parameters():
            prm.copy_(_bf(prm.shape, g, 0.08))
    x = _bf((1, 203, 128), g)
    types = torch.rand(1, 203, generator=g) > 0.7
    dy = _bf((1, 203, 128), g)
    nw = (1.0 + 0.1 * torch.randn(128, generator=g)).to(torch.bfloat16)
    # reference: fp32 leaves, oracle forward, torch autograd
    xr = x.float().requires_grad_(True)
    wr = [tuple(w.detach().float().requires_grad_(True) for w in e.weights()) for e in block.experts]
    hin = oracle.rms_norm_ref(xr, nw.float(), 1e-6) if fused_extras else xr
    yr = oracle.sparse_moe_block_ref(hin, types, wr, eager_rounding=False)
    if fused_extras:
        yr = xr + yr
    yr.backward(dy.float())
    # kernels
    block = block.to(dev)
    xd = x.to(dev).requires_grad_(True)
    kw = dict(pre_norm=(nw.to(dev), 1e-6), residual=True) if fused_extras else {}
    yd = block(xd, types.to(dev), **kw)
    _close(yd, yr.detach(), atol=3e-2, rtol=2e-2, what="forward under autograd")
    yd.backward(dy.to(dev))
    _close(xd.grad, xr.grad, atol=3e-2, rtol=3e-2, what="grad of the input")
    for e in range(2):
        for name, wref in zip(("gate", "up", "down"), wr[e]):
            got = getattr(block.experts[e], f"{name}_proj").weight.grad
            scale = float(wref.grad.abs().max())
            err = float((got.float().cpu() - wref.grad).abs().max())
            assert err <= 0.03 * scale + 1e-3, f"expert {e} {name}: max err {err} at scale {scale}"
