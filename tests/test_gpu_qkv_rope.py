"""GPU parity of the q / k / v projection with M-RoPE in the GEMM epilogue (vl.py:955-964 as one launch) against the
oracle: an fp32 linear layer rounded to bf16, then mrope_apply_ref in eager bf16, in both channel layouts (the
PyTorch path's, vl.py:763-769, and the CUDA kernel's, csrc/rope.cu:104-117, which the flash-attention class of
vl.py:962-964 runs).  Tolerance |x - ref| <= 2e-2 + 1e-2 |ref|."""

import pytest
import torch
import torch.nn.functional as F

import oracle
from wallx_mi355 import _lib, native, workloads as wl
from wallx_mi355.fusions import ops

pytestmark = pytest.mark.gpu


def _close(got, ref, what):
    got, ref = got.float().cpu(), ref.float()
    assert got.shape == ref.shape, what
    err = (got - ref).abs()
    bad = err > 2e-2 + 1e-2 * ref.abs()
    assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance, max abs err {float(err.max())}"


def _reference(x, w, b, pos, nq, nkv, rows=None, layout="hf"):
    """(q, k, v) [B, H, S, D] from the oracle; rows: optional token subset (flattened indices) to evaluate."""
    B, S, H = x.shape
    D = 128
    xf = x.reshape(B * S, H)
    cos, sin = oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(), torch.bfloat16)
    if rows is not None:
        xf = xf[rows]
        cos = cos.reshape(3, 1, B * S, D)[:, :, rows]
        sin = sin.reshape(3, 1, B * S, D)[:, :, rows]
        B, S = 1, rows.numel()
    qkv = F.linear(xf.float(), w.float(), None if b is None else b.float()).to(torch.bfloat16)
    q, k, v = qkv.split([nq * D, nkv * D, nkv * D], dim=-1)
    q = q.reshape(B, S, nq, D).transpose(1, 2)
    k = k.reshape(B, S, nkv, D).transpose(1, 2)
    v = v.reshape(B, S, nkv, D).transpose(1, 2)
    rq, rk = oracle.mrope_apply_ref(q, k, cos, sin, list(wl.MROPE_SECTION), layout, eager_rounding=True)
    return rq, rk, v


@pytest.mark.parametrize("layout", ["hf", "csrc"])
@pytest.mark.parametrize("B,S,H,nq,nkv,with_bias", [(2, 300, 512, 4, 2, True), (1, 37, 256, 2, 1, False),
                                                   (3, 256, 1024, 3, 1, True), (1, 1, 64, 1, 1, True)])
def test_qkv_rope_projection(dev, B, S, H, nq, nkv, with_bias, layout):
    g = torch.Generator().manual_seed(B * 1000 + S)
    x = torch.randn(B, S, H, generator=g).to(torch.bfloat16)
    n = (nq + 2 * nkv) * 128
    w = (torch.randn(n, H, generator=g) * 0.05).to(torch.bfloat16)
    b = (torch.randn(n, generator=g) * 0.5).to(torch.bfloat16) if with_bias else None
    pos = torch.stack([torch.randint(0, 60, (B, S), generator=g), torch.randint(100, 160, (B, S), generator=g),
                       torch.randint(300, 360, (B, S), generator=g)])  # distinct planes
    width = 64 if layout == "hf" else 128  # the CUDA kernel's layout rotates d and d + 64 by different planes
    table = ops.multimodal_rope_table(pos.to(dev), wl.text_inv_freq().to(dev), wl.MROPE_SECTION, layout)
    assert table.shape == (B * S, width) and table.dtype == torch.int32
    # the table itself: bf16 cos / sin of the oracle's builder, packed
    cos, sin = oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(), torch.bfloat16)
    amap = oracle.mrope_axis_map(wl.MROPE_SECTION, 128, layout)[:width]
    cos_sel = cos[amap, :, :, torch.arange(width)].permute(1, 2, 0).reshape(B * S, width)
    sin_sel = sin[amap, :, :, torch.arange(width)].permute(1, 2, 0).reshape(B * S, width)
    tb = table.cpu()
    got_cos = (tb << 16).view(torch.float32)
    got_sin = (tb & -65536).view(torch.float32)
    assert float((got_cos != cos_sel.float()).float().mean()) < 5e-3  # sincosf of the device vs the host: a bf16 step now and then
    assert float((got_sin != sin_sel.float()).float().mean()) < 5e-3
    assert bool(((got_cos - cos_sel.float()).abs() <= 2.0 ** -7).all()) and bool(((got_sin - sin_sel.float()).abs() <= 2.0 ** -7).all())
    q, k, v = ops.qkv_projection_with_rope(x.to(dev), w.to(dev), None if b is None else b.to(dev), table, nq, nkv)
    assert q.shape == (B, nq, S, 128) and k.shape == (B, nkv, S, 128) and v.shape == (B, nkv, S, 128)
    rq, rk, rv = _reference(x, w, b, pos, nq, nkv, layout=layout)
    if layout == "csrc":  # the two layouts must not coincide on these positions (distinct planes)
        hq, _, _ = _reference(x, w, b, pos, nq, nkv, layout="hf")
        assert not torch.equal(hq, rq)
    _close(q, rq, "q")
    _close(k, rk, "k")
    _close(v, rv, "v")
    # the same numbers as the two-step path on the device (projection by torch, then the rope kernel from positions)
    qkv = F.linear(x.to(dev), w.to(dev), None if b is None else b.to(dev))
    q2, k2, _ = qkv.split([nq * 128, nkv * 128, nkv * 128], dim=-1)
    gq, gk = ops.multimodal_rope_from_positions(q2.reshape(B, S, nq, 128).transpose(1, 2), k2.reshape(B, S, nkv, 128).transpose(1, 2),
                                                pos.to(dev), wl.text_inv_freq().to(dev), list(wl.MROPE_SECTION), layout)
    _close(q, gq.cpu(), "q vs two-step path")
    _close(k, gk.cpu(), "k vs two-step path")


def test_qkv_rope_projection_config5_shape(dev):
    """The prefill shape: 16 x 912 tokens, hidden 2048, 16 query and 2 KV heads (N = 2560); the oracle on a sample of
    tokens, every column."""
    ids, grid = wl.config2_tokens(batch=16, tail_text=96)
    pos, _ = oracle.rope_index_ref(ids, 2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, 2,
                                   image_grid_thw=grid)
    B, S = ids.shape
    g = torch.Generator().manual_seed(7)
    x = torch.randn(B, S, 2048, generator=g).to(torch.bfloat16)
    w = (torch.randn(2560, 2048, generator=g) * 0.02).to(torch.bfloat16)
    b = (torch.randn(2560, generator=g) * 0.02).to(torch.bfloat16)
    table = ops.multimodal_rope_table(pos.to(dev), wl.text_inv_freq().to(dev), wl.MROPE_SECTION)
    q, k, v = ops.qkv_projection_with_rope(x.to(dev), w.to(dev), b.to(dev), table, 16, 2)
    rows = torch.cat([torch.arange(0, B * S, 97), torch.tensor([B * S - 1])])  # spread over every row tile
    rq, rk, rv = _reference(x, w, b, pos, 16, 2, rows)
    pick = lambda t: t.transpose(1, 2).reshape(B * S, -1, 128)[rows.to(dev)].cpu()  # noqa: E731  [rows, heads, D]
    _close(pick(q), rq[0].transpose(0, 1), "q sample")
    _close(pick(k), rk[0].transpose(0, 1), "k sample")
    _close(pick(v), rv[0].transpose(0, 1), "v sample")


def test_qkv_rope_rejects_what_it_cannot_do(dev):
    lib = _lib.load()
    pos = torch.zeros(3, 1, 4, dtype=torch.int64, device=dev)
    p = pos.data_ptr()
    assert lib.wx_qkv_rope_proj(p, p, None, p, 32, p, 4, 64, 1, 1, 64, None) == -2
    assert b"head_dim" in lib.wx_last_error_string()


@pytest.mark.parametrize("layout", ["hf", "csrc"])
@pytest.mark.parametrize("B,S,H,nq,nkv,with_bias", [(2, 200, 512, 4, 2, True), (1, 37, 256, 2, 1, False)])
def test_qkv_rope_projection_backward(dev, B, S, H, nq, nkv, with_bias, layout):
    """Gradients of the fused projection against torch autograd of the fp32 expression it fuses (linear, then the
    oracle's M-RoPE in fp32 on the same cos / sin): d hidden, d weight, d bias for a random cotangent on q, k and v.
    The fused op rounds the forward and the rotated gradient to bf16 like the eager bf16 path, so the comparison
    carries the GEMM tolerance, scaled to each gradient's magnitude."""
    g = torch.Generator().manual_seed(B * 77 + S)
    D = 128
    n = (nq + 2 * nkv) * D
    x = torch.randn(B, S, H, generator=g).to(torch.bfloat16)
    w = (torch.randn(n, H, generator=g) * 0.05).to(torch.bfloat16)
    b = (torch.randn(n, generator=g) * 0.5).to(torch.bfloat16) if with_bias else None
    pos = torch.stack([torch.randint(0, 60, (B, S), generator=g), torch.randint(100, 160, (B, S), generator=g),
                       torch.randint(300, 360, (B, S), generator=g)])
    cq = torch.randn(B, nq, S, D, generator=g).to(torch.bfloat16)
    ck = torch.randn(B, nkv, S, D, generator=g).to(torch.bfloat16)
    cv = torch.randn(B, nkv, S, D, generator=g).to(torch.bfloat16)
    # reference: fp32 autograd through linear and the oracle's rotation
    xr, wr = x.float().requires_grad_(True), w.float().requires_grad_(True)
    br = None if b is None else b.float().requires_grad_(True)
    cos, sin = oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(), torch.bfloat16)
    qkv = F.linear(xr, wr, br)
    q, k, v = qkv.split([nq * D, nkv * D, nkv * D], dim=-1)
    q = q.reshape(B, S, nq, D).transpose(1, 2)
    k = k.reshape(B, S, nkv, D).transpose(1, 2)
    v = v.reshape(B, S, nkv, D).transpose(1, 2)
    rq, rk = oracle.mrope_apply_ref(q, k, cos.float(), sin.float(), list(wl.MROPE_SECTION), layout)
    ((rq * cq.float()).sum() + (rk * ck.float()).sum() + (v * cv.float()).sum()).backward()
    # fused op
    xd, wd = x.to(dev).requires_grad_(True), w.to(dev).requires_grad_(True)
    bd = None if b is None else b.to(dev).requires_grad_(True)
    table = ops.multimodal_rope_table(pos.to(dev), wl.text_inv_freq().to(dev), wl.MROPE_SECTION, layout)
    gq, gk, gv = ops.qkv_projection_with_rope(xd, wd, bd, table, nq, nkv, mrope_section=wl.MROPE_SECTION)
    torch.autograd.backward([gq, gk, gv], [cq.to(dev), ck.to(dev), cv.to(dev)])

    def close(got, ref, what):
        got, ref = got.float().cpu(), ref.float()
        s = float(ref.pow(2).mean().sqrt())
        bad = (got - ref).abs() > 2e-2 * s + 1e-2 * ref.abs()
        assert not bad.any(), f"{what}: {int(bad.sum())} of {bad.numel()} outside tolerance (rms {s})"

    close(xd.grad, xr.grad, "d hidden_states")
    close(wd.grad, wr.grad, "d qkv_weight")
    if b is not None:
        close(bd.grad, br.grad, "d qkv_bias")
    # the forward under autograd is the same launch as without it
    with torch.no_grad():
        q0, k0, v0 = ops.qkv_projection_with_rope(x.to(dev), w.to(dev), None if b is None else b.to(dev), table, nq, nkv)
    assert torch.equal(q0, gq) and torch.equal(k0, gk) and torch.equal(v0, gv)
