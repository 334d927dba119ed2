"""RMSNorm + tiled permute and unpermute + residual add (the caller fusions around the FFN) against the oracle."""

import pytest
import torch

import oracle
from wallx_mi355 import moe, native

pytestmark = pytest.mark.gpu


def _bf(shape, g, std=1.0):
    return (torch.randn(shape, generator=g) * std).to(torch.bfloat16)


def _untile(tiled, rows_pad, H):
    """K-tiled [rows_pad, H] (16 x 32 blocks, [column block][row block], swizzled 16-byte chunks) -> row-major."""
    rb, kb = rows_pad // 16, H // 32
    t = tiled[: rows_pad * H].view(kb, rb, 16, 4, 8)
    out = torch.empty(rows_pad, H, dtype=tiled.dtype)
    for r in range(16):
        for c in range(4):
            slot = c ^ ((r >> 2) & 3)
            out.view(rb, 16, kb, 4, 8)[:, r, :, c, :] = t[:, :, r, slot, :].transpose(0, 1)
    return out


@pytest.mark.parametrize("T,H,n_act", [(300, 256, 37), (912, 2048, 32), (64, 128, 0), (50, 4096, 50), (1000, 1536, 999)])
def test_rmsnorm_permute_tiled(dev, T, H, n_act):
    g = torch.Generator().manual_seed(T + H)
    x = _bf((T, H), g, 3.0)
    w = (1.0 + 0.1 * torch.randn(H, generator=g)).to(torch.bfloat16)
    types = torch.zeros(T, dtype=torch.bool)
    types[torch.randperm(T, generator=g)[:n_act]] = True
    rmap, off, inv, _ = native.partition(types.to(dev), 2, 0, None, want_sorted=True)
    fused = native.rmsnorm_permute_rows_tiled(x.to(dev), w.to(dev), 1e-6, off, inv)
    # the same layout from the unfused pair, fed with the oracle's norm: equal except where the fp32 sum of squares
    # (accumulated in a different order) moves a value across a rounding boundary
    normed = oracle.rms_norm_ref(x, w, 1e-6)
    plain = native.permute_rows_tiled(normed.to(dev), rmap, off, None, inv)
    rows_pad = native.padded_sorted_rows(T)
    a = _untile(fused.cpu(), rows_pad, H).float()
    b = _untile(plain.cpu(), rows_pad, H).float()
    o = off.cpu().tolist()
    pad0 = (o[1] + 255) // 256 * 256
    live = torch.zeros(rows_pad, dtype=torch.bool)
    live[: o[1]] = True
    live[pad0: pad0 + (o[2] - o[1])] = True
    a, b = a[live], b[live]
    assert a.shape[0] == T
    # one bf16 step in the normalised value, which its rounded product with the weight can turn into two
    bad = (a - b).abs() > 2.0 ** -6 * b.abs() + 1e-6
    assert not bad.any(), f"{int(bad.sum())} of {bad.numel()} differ by more than two bf16 steps"
    one = (a - b).abs() > 2.0 ** -7 * b.abs() + 1e-6
    assert float(one.float().mean()) < 1e-4  # more than one step: a handful per million
    assert float((a != b).float().mean()) < 0.02  # and almost all values are identical


@pytest.mark.parametrize("T,H", [(300, 256), (912, 2048), (7, 8), (33, 1000)])
def test_unpermute_add(dev, T, H):
    g = torch.Generator().manual_seed(T * H)
    y, resid = _bf((T, H), g), _bf((T, H), g)
    types = torch.rand(T, generator=g) < 0.2
    _, rmap_ref, _ = oracle.permute_ref(y, types)
    rmap, _, _, _ = native.partition(types.to(dev), 2, 0, None, want_sorted=False)
    got = native.unpermute_add(y.to(dev), resid.to(dev), rmap)
    ref = resid + oracle.unpermute_ref(y, rmap_ref)  # eager bf16 add: one rounding
    assert torch.equal(got.cpu(), ref)


@pytest.mark.parametrize("T,H", [(300, 256), (912, 2048), (7, 8), (33, 1000), (20, 4096)])
def test_unpermute_add_rmsnorm(dev, T, H):
    """The closing residual add of a layer with the next reader's RMSNorm in the same pass: the sum is bit-equal to
    the eager add; the norm equals the oracle's RMSNorm of that (bf16) sum except where the fp32 sum of squares,
    accumulated in another order, moves the normalised value across a rounding boundary: one bf16 step there, which
    the rounded product with the weight can turn into two."""
    g = torch.Generator().manual_seed(T * H + 1)
    y, resid = _bf((T, H), g, 2.0), _bf((T, H), g, 2.0)
    w = (1.0 + 0.1 * torch.randn(H, generator=g)).to(torch.bfloat16)
    types = torch.rand(T, generator=g) < 0.2
    _, rmap_ref, _ = oracle.permute_ref(y, types)
    rmap, _, _, _ = native.partition(types.to(dev), 2, 0, None, want_sorted=False)
    out, normed = native.unpermute_add_rmsnorm(y.to(dev), resid.to(dev), rmap, w.to(dev), 1e-6)
    ref_sum = resid + oracle.unpermute_ref(y, rmap_ref)
    assert torch.equal(out.cpu(), ref_sum)
    ref_norm = oracle.rms_norm_ref(ref_sum, w, 1e-6).float()
    got = normed.cpu().float()
    bad = (got - ref_norm).abs() > 2.0 ** -6 * ref_norm.abs() + 1e-6
    assert not bad.any(), f"{int(bad.sum())} of {bad.numel()} differ by more than two bf16 steps"
    one = (got - ref_norm).abs() > 2.0 ** -7 * ref_norm.abs() + 1e-6
    assert float(one.float().mean()) < 1e-4  # more than one step: a handful per million
    assert float((got != ref_norm).float().mean()) < 0.02


@pytest.mark.parametrize("T,H,n_act", [(300, 256, 37), (912, 2048, 32), (7, 8, 7), (33, 1000, 0), (20, 4096, 11)])
def test_rmsnorm_permute_rows(dev, T, H, n_act):
    """The normed rows in expert-sorted order, row-major: the oracle's RMSNorm followed by its permute, up to the
    rounding-boundary steps the fp32 sum of squares (another accumulation order) allows."""
    g = torch.Generator().manual_seed(T + 3 * H)
    x = _bf((T, H), g, 2.0)
    w = (1.0 + 0.1 * torch.randn(H, generator=g)).to(torch.bfloat16)
    types = torch.zeros(T, dtype=torch.bool)
    types[torch.randperm(T, generator=g)[:n_act]] = True
    ref, _, _ = oracle.permute_ref(oracle.rms_norm_ref(x, w, 1e-6), types)
    _, _, inv, _ = native.partition(types.to(dev), 2, 0, None, want_sorted=True)
    got = native.rmsnorm_permute_rows(x.to(dev), w.to(dev), 1e-6, inv).cpu().float()
    ref = ref.float()
    bad = (got - ref).abs() > 2.0 ** -6 * ref.abs() + 1e-6
    assert not bad.any(), f"{int(bad.sum())} of {bad.numel()} differ by more than two bf16 steps"
    assert float((got != ref).float().mean()) < 0.02


@pytest.mark.parametrize("with_add", [False, True])
@pytest.mark.parametrize("T,H,n_act", [(300, 256, 37), (912, 2048, 32), (7, 8, 7), (33, 1000, 0), (3000, 1024, 800)])
def test_unpermute_rmsnorm_bwd(dev, T, H, n_act, with_add):
    """Backward of permute(weight * rmsnorm(x)) for a gradient of the sorted rows, against torch autograd of the
    oracle's RMSNorm and permute in fp32 (the kernel rounds its result once, to bf16): the input gradient, with and
    without the residual branch's gradient summed in, and the weight gradient."""
    g = torch.Generator().manual_seed(T * 7 + H)
    x = _bf((T, H), g, 2.0)
    w = (1.0 + 0.1 * torch.randn(H, generator=g)).to(torch.bfloat16)
    gs = _bf((T, H), g)  # gradient w.r.t. the sorted, normed rows
    add = _bf((T, H), g) if with_add else None
    types = torch.zeros(T, dtype=torch.bool)
    types[torch.randperm(T, generator=g)[:n_act]] = True
    xr, wr = x.float().requires_grad_(True), w.float().requires_grad_(True)
    sorted_ref, _, _ = oracle.permute_ref(oracle.rms_norm_ref(xr, wr, 1e-6), types)
    loss = (sorted_ref * gs.float()).sum()
    if with_add:
        loss = loss + (xr * add.float()).sum()
    loss.backward()
    rmap, _, _, _ = native.partition(types.to(dev), 2, 0, None, want_sorted=False)
    gx, gw = native.unpermute_rmsnorm_bwd(gs.to(dev), x.to(dev), w.to(dev), 1e-6, rmap,
                                          add=None if add is None else add.to(dev))
    ref = xr.grad
    err = (gx.cpu().float() - ref).abs()
    assert not (err > 2.0 ** -7 * ref.abs() + 2e-3 * float(ref.abs().mean())).any(), float(err.max())
    scale = float(wr.grad.abs().max())
    werr = float((gw.cpu().float() - wr.grad).abs().max())
    assert werr <= 2.0 ** -7 * scale + 1e-3 * scale, f"weight gradient: max err {werr} at scale {scale}"


def test_moe_block_with_both_fusions(dev):
    """h + block(RMSNorm(h)) through the module's fused path against the same module fed by separate PyTorch ops."""
    from types import SimpleNamespace

    g = torch.Generator().manual_seed(11)
    cfg = SimpleNamespace(experts=[dict(hidden_size=256, intermediate_size=512, hidden_act="silu"),
                                   dict(hidden_size=256, intermediate_size=128, hidden_act="silu")])
    block = moe.SparseMoeBlock(cfg, 2).to(dev).to(torch.bfloat16)
    with torch.no_grad():
        for prm in block.parameters():
            prm.copy_((torch.randn(prm.shape, generator=g) * 0.05).to(torch.bfloat16))
    h = _bf((2, 150, 256), g, 2.0).to(dev)
    w = (1.0 + 0.1 * torch.randn(256, generator=g)).to(torch.bfloat16).to(dev)
    types = (torch.rand(2, 150, generator=g) < 0.1).to(dev)
    with torch.no_grad():
        fused = block(h, types, pre_norm=(w, 1e-6), residual=True)
        plain = h + block(oracle.rms_norm_ref(h.cpu(), w.cpu(), 1e-6).to(dev), types)
    err = (fused.float() - plain.float()).abs()
    assert not (err > 2e-2 + 1e-2 * plain.float().abs()).any(), float(err.max())


@pytest.mark.parametrize("with_norm,with_residual", [(False, False), (True, False), (False, True), (True, True)])
def test_block_forward_as_one_library_call_equals_its_launches(dev, with_norm, with_residual):
    """wx_moe_block_forward through the C ABI against the entry points it is made of, called one by one on buffers of
    their own: bit-equal, with and without the fused RMSNorm and residual add."""
    from wallx_mi355 import _lib

    g = torch.Generator().manual_seed(31)
    T, H, I0, I1 = 700, 256, 384, 128
    x = _bf((T, H), g, 2.0).to(dev)
    nw = (1.0 + 0.1 * torch.randn(H, generator=g)).to(torch.bfloat16).to(dev)
    types = (torch.rand(T, generator=g) < 0.2).to(dev)
    ws = [(torch.randn(s, generator=g) * 0.05).to(torch.bfloat16).to(dev)
          for s in ((I0, H), (I0, H), (H, I0), (I1, H), (I1, H), (H, I1))]
    packed = [native.pack_weight(w, cache=False) for w in ws]
    rmap, off, inv, _ = native.partition(types, 2, 0, None, want_sorted=True)
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    pad = native.padded_sorted_rows(T)
    bufs = [(torch.empty(lib.wx_tiled_bytes(pad, H) // 2, dtype=torch.bfloat16, device=dev),
             torch.empty(pad * max(I0, I1), dtype=torch.bfloat16, device=dev), torch.empty_like(x)) for _ in range(2)]
    (xt, hm, out), (xt2, hm2, out2) = bufs
    p = [t.data_ptr() for t in packed]
    eps = 1e-6
    _lib.call("wx_moe_block_forward", x.data_ptr(), out.data_ptr(), rmap.data_ptr(), inv.data_ptr(), off.data_ptr(),
              p[0], p[1], p[2], p[3], p[4], p[5], xt.data_ptr(), hm.data_ptr(), T, H, I0, I1, None,
              nw.data_ptr() if with_norm else None, eps, int(with_residual), None, stream)
    if with_norm:
        _lib.call("wx_rmsnorm_permute_rows_tiled", x.data_ptr(), nw.data_ptr(), eps, xt2.data_ptr(), inv.data_ptr(),
                  off.data_ptr(), T, H, stream)
    else:
        _lib.call("wx_permute_rows_tiled", x.data_ptr(), xt2.data_ptr(), rmap.data_ptr(), inv.data_ptr(),
                  off.data_ptr(), T, H, stream)
    _lib.call("wx_dual_swiglu_gate_up", xt2.data_ptr(), hm2.data_ptr(), off.data_ptr(), p[0], p[1], p[3], p[4], T, H,
              I0, I1, None, stream)
    if with_residual:
        _lib.call("wx_dual_down_proj_residual", hm2.data_ptr(), out2.data_ptr(), x.data_ptr(), off.data_ptr(), p[2],
                  p[5], T, H, I0, I1, None, inv.data_ptr(), stream)
    else:
        _lib.call("wx_dual_down_proj", hm2.data_ptr(), out2.data_ptr(), off.data_ptr(), p[2], p[5], T, H, I0, I1, None,
                  inv.data_ptr(), stream)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)
    # and against the oracle
    hin = oracle.rms_norm_ref(x.cpu(), nw.cpu(), eps) if with_norm else x.cpu()
    wc = [tuple(w.cpu() for w in ws[:3]), tuple(w.cpu() for w in ws[3:])]
    ref = oracle.sparse_moe_block_ref(hin[None], types.cpu()[None], wc)[0].float()
    if with_residual:
        ref = (x.cpu().float() + ref).to(torch.bfloat16).float()
    err = (out.cpu().float() - ref).abs()
    assert not (err > 2e-2 + 1e-2 * ref.abs()).any(), float(err.max())
    assert lib.wx_moe_block_forward(x.data_ptr(), out.data_ptr(), rmap.data_ptr(), None, off.data_ptr(), p[0], p[1],
                                    p[2], p[3], p[4], p[5], xt.data_ptr(), hm.data_ptr(), T, H, I0, I1, None, None,
                                    eps, 0, None, stream) == -1  # sorted_row_id is required
