"""GPU parity: 3D M-RoPE apply against the oracle (eager bf16 evaluation of vl.py:731-773)."""

import warnings

import pytest
import torch

import oracle
from wallx_mi355 import native, workloads as wl
from wallx_mi355.fusions import ops

pytestmark = pytest.mark.gpu

ATOL, RTOL = 2e-2, 1e-2  # |x - ref| <= 2e-2 + 1e-2 |ref| for bf16 outputs


def _close(got, ref, atol=ATOL, rtol=RTOL):
    got, ref = got.float().cpu(), ref.float()
    bad = (got - ref).abs() > atol + rtol * ref.abs()
    assert not bad.any(), f"{int(bad.sum())} of {bad.numel()} outside tolerance, max abs {float((got - ref).abs().max())}"


def _n_diff(got, ref):
    return int((got.cpu() != ref).sum())


def _inputs(B, S, dtype, seed, hq=4, hk=2):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, S, hq, 128, generator=g).to(dtype)
    k = torch.randn(B, S, hk, 128, generator=g).to(dtype)
    pos = torch.randint(0, 2000, (3, B, S), generator=g)
    cos, sin = oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(), dtype)
    return q, k, cos, sin


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("layout", ["hf", "csrc"])
def test_mrope_matches_eager_bit_for_bit(dev, dtype, layout):
    q, k, cos, sin = _inputs(2, 37, dtype, 5)
    qt, kt = q.transpose(1, 2), k.transpose(1, 2)  # [B, H, S, D] views of token-major memory
    rq, rk = oracle.mrope_apply_ref(qt, kt, cos, sin, list(wl.MROPE_SECTION), layout, eager_rounding=True)
    gq, gk = ops.multimodal_rope(qt.to(dev), kt.to(dev), cos.to(dev), sin.to(dev), list(wl.MROPE_SECTION), layout)
    assert gq.shape == rq.shape and gq.is_contiguous() and gk.is_contiguous()
    _close(gq, rq)
    _close(gk, rk)
    if dtype != torch.float16:
        # the kernel rounds each product and the sum exactly like eager evaluation, so the match is exact
        # (fp16 on the host may use native half arithmetic, whose sum is rounded once instead of twice)
        assert _n_diff(gq, rq) == 0 and _n_diff(gk, rk) == 0
    else:
        _close(gq, rq, atol=2e-3, rtol=2e-3)


def test_mrope_strided_views_need_no_copy(dev):
    q, k, cos, sin = _inputs(3, 20, torch.bfloat16, 7)
    qd, kd = q.to(dev), k.to(dev)
    with warnings.catch_warnings():
        warnings.simplefilter("error")  # no "discontiguous" warning: strided [B,H,S,D] views are read in place
        gq, gk = ops.multimodal_rope(qd.transpose(1, 2), kd.transpose(1, 2), cos.to(dev), sin.to(dev), [16, 24, 24])
    cq, ck = ops.multimodal_rope(qd.transpose(1, 2).contiguous(), kd.transpose(1, 2).contiguous(), cos.to(dev),
                                 sin.to(dev), [16, 24, 24])
    assert _n_diff(gq, cq.cpu()) == 0 and _n_diff(gk, ck.cpu()) == 0


def test_mrope_config2_full_size(dev):
    """B = 16, S = 896, q [14336,16,128], k [14336,2,128] bf16 with the real position ids of the layout."""
    ids, grid = wl.config2_tokens()
    pos, _ = oracle.rope_index_ref(ids, 2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, 2,
                                   image_grid_thw=grid)
    cos, sin = oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(), torch.bfloat16)
    q, k = wl.qk_inputs(16, 896)
    qt, kt = q.transpose(1, 2), k.transpose(1, 2)
    rq, rk = oracle.mrope_apply_ref(qt, kt, cos, sin, list(wl.MROPE_SECTION), "hf")
    gq, gk = ops.multimodal_rope(qt.to(dev), kt.to(dev), cos.to(dev), sin.to(dev), list(wl.MROPE_SECTION))
    _close(gq, rq)
    _close(gk, rk)
    assert _n_diff(gq, rq) == 0 and _n_diff(gk, rk) == 0
    # fp32-math oracle (one rounding) is within the stated tolerance as well
    fq, fk = oracle.mrope_apply_ref(qt, kt, cos, sin, list(wl.MROPE_SECTION), "hf", eager_rounding=False)
    _close(gq, fq)
    # rotation pairs (d, d + 64) keep their norm up to bf16 rounding
    n_in = (qt[..., :64].float() ** 2 + qt[..., 64:].float() ** 2)
    n_out = (gq[..., :64].float().cpu() ** 2 + gq[..., 64:].float().cpu() ** 2)
    assert torch.all((n_in - n_out).abs() <= 0.05 * n_in + 0.05)


def test_mrope_non_multiple_of_8_sections(dev):
    q, k, cos, sin = _inputs(1, 9, torch.bfloat16, 9)
    sec = [10, 27, 27]
    rq, rk = oracle.mrope_apply_ref(q.transpose(1, 2), k.transpose(1, 2), cos, sin, sec, "hf")
    gq, gk = ops.multimodal_rope(q.transpose(1, 2).to(dev), k.transpose(1, 2).to(dev), cos.to(dev), sin.to(dev), sec)
    assert _n_diff(gq, rq) == 0 and _n_diff(gk, rk) == 0
    with pytest.raises(RuntimeError, match="covers"):
        ops.multimodal_rope(q.transpose(1, 2).to(dev), k.transpose(1, 2).to(dev), cos.to(dev), sin.to(dev), [16, 24, 20])


@pytest.mark.parametrize("layout", ["hf", "csrc"])
def test_mrope_backward(dev, layout):
    q, k, cos, sin = _inputs(2, 11, torch.float32, 13)
    qd = q.transpose(1, 2).to(dev).requires_grad_(True)
    kd = k.transpose(1, 2).to(dev).requires_grad_(True)
    oq, ok = ops.multimodal_rope(qd, kd, cos.to(dev), sin.to(dev), list(wl.MROPE_SECTION), layout)
    g = torch.Generator().manual_seed(3)
    gq, gk = torch.randn(oq.shape, generator=g), torch.randn(ok.shape, generator=g)
    torch.autograd.backward([oq, ok], [gq.to(dev), gk.to(dev)])
    rq, rk = oracle.mrope_apply_bwd_ref(gq, gk, cos, sin, list(wl.MROPE_SECTION), layout)
    assert torch.allclose(qd.grad.cpu(), rq, rtol=1e-5, atol=1e-5)
    assert torch.allclose(kd.grad.cpu(), rk, rtol=1e-5, atol=1e-5)


# ----------------------------------------------------------------------------- cos/sin evaluated in the kernel
def _pos_inputs(B, S, dtype, seed, hq=4, hk=2, max_pos=2000):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, S, hq, 128, generator=g).to(dtype)
    k = torch.randn(B, S, hk, 128, generator=g).to(dtype)
    pos = torch.randint(0, max_pos, (3, B, S), generator=g)
    return q, k, pos


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("layout", ["hf", "csrc"])
def test_mrope_from_positions_matches_the_table_path(dev, dtype, layout):
    """The oracle builds the tables (fp32 angle, fp32 cos/sin, cast: vl.py:679-712) and rotates; the kernel gets
    only position_ids and inv_freq.  The device's sincosf and the host's differ in the last place now and then, so a
    rounded table entry may differ by one unit of the storage type: stated tolerance everywhere, and all but a
    sliver of the outputs bit-equal."""
    q, k, pos = _pos_inputs(2, 61, dtype, 21)
    inv_freq = wl.text_inv_freq()
    cos, sin = oracle.rotary_cos_sin_ref(pos, inv_freq, dtype)
    qt, kt = q.transpose(1, 2), k.transpose(1, 2)
    rq, rk = oracle.mrope_apply_ref(qt, kt, cos, sin, list(wl.MROPE_SECTION), layout, eager_rounding=True)
    gq, gk = ops.multimodal_rope_from_positions(qt.to(dev), kt.to(dev), pos.to(dev), inv_freq.to(dev),
                                                list(wl.MROPE_SECTION), layout)
    assert gq.is_contiguous() and gk.is_contiguous()
    if dtype == torch.float32:
        # fp32 tables keep the full last-place difference; angles reach 2000 rad, where one ulp of the angle is 1e-4
        _close(gq, rq, atol=1e-3, rtol=1e-3)
        _close(gk, rk, atol=1e-3, rtol=1e-3)
    else:
        _close(gq, rq)
        _close(gk, rk)
        assert _n_diff(gq, rq) <= 2e-3 * rq.numel() and _n_diff(gk, rk) <= 2e-3 * rk.numel()


def test_mrope_from_positions_config2_full_size(dev):
    ids, grid = wl.config2_tokens()
    pos, _ = oracle.rope_index_ref(ids, 2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, 2,
                                   image_grid_thw=grid)
    inv_freq = wl.text_inv_freq()
    cos, sin = oracle.rotary_cos_sin_ref(pos, inv_freq, torch.bfloat16)
    q, k = wl.qk_inputs(16, 896)
    qt, kt = q.transpose(1, 2), k.transpose(1, 2)
    rq, rk = oracle.mrope_apply_ref(qt, kt, cos, sin, list(wl.MROPE_SECTION), "hf")
    gq, gk = ops.multimodal_rope_from_positions(qt.to(dev), kt.to(dev), pos.to(dev), inv_freq.to(dev),
                                                list(wl.MROPE_SECTION))
    _close(gq, rq)
    _close(gk, rk)
    assert _n_diff(gq, rq) <= 1e-3 * rq.numel() and _n_diff(gk, rk) <= 1e-3 * rk.numel()
    # position 0 on every axis is the identity whatever the frequencies: cos = 1, sin = 0 exactly
    zero = torch.zeros_like(pos)
    iq, ik = ops.multimodal_rope_from_positions(qt.to(dev), kt.to(dev), zero.to(dev), inv_freq.to(dev),
                                                list(wl.MROPE_SECTION))
    assert _n_diff(iq, qt.contiguous()) == 0 and _n_diff(ik, kt.contiguous()) == 0


def test_mrope_from_positions_backward_is_the_adjoint(dev):
    q, k, pos = _pos_inputs(2, 11, torch.float32, 23, max_pos=300)
    inv_freq = wl.text_inv_freq()
    cos, sin = oracle.rotary_cos_sin_ref(pos, inv_freq, torch.float32)
    qd = q.transpose(1, 2).to(dev).requires_grad_(True)
    kd = k.transpose(1, 2).to(dev).requires_grad_(True)
    oq, ok = ops.multimodal_rope_from_positions(qd, kd, pos.to(dev), inv_freq.to(dev), list(wl.MROPE_SECTION))
    g = torch.Generator().manual_seed(3)
    gq, gk = torch.randn(oq.shape, generator=g), torch.randn(ok.shape, generator=g)
    torch.autograd.backward([oq, ok], [gq.to(dev), gk.to(dev)])
    rq, rk = oracle.mrope_apply_bwd_ref(gq, gk, cos, sin, list(wl.MROPE_SECTION), "hf")
    assert torch.allclose(qd.grad.cpu(), rq, rtol=1e-4, atol=1e-4)
    assert torch.allclose(kd.grad.cpu(), rk, rtol=1e-4, atol=1e-4)
    # <forward(x), g> == <x, backward(g)>
    lhs = float((oq.detach().cpu().double() * gq.double()).sum() + (ok.detach().cpu().double() * gk.double()).sum())
    rhs = float((qd.grad.cpu().double() * q.transpose(1, 2).double()).sum()
                + (kd.grad.cpu().double() * k.transpose(1, 2).double()).sum())
    assert abs(lhs - rhs) <= 1e-3 * max(1.0, abs(lhs))


def test_mrope_from_positions_refuses_what_it_cannot_do(dev):
    q, k, pos = _pos_inputs(1, 9, torch.bfloat16, 9)
    inv_freq = wl.text_inv_freq().to(dev)
    with pytest.raises(RuntimeError, match="chunk boundaries"):
        ops.multimodal_rope_from_positions(q.transpose(1, 2).to(dev), k.transpose(1, 2).to(dev), pos.to(dev), inv_freq,
                                           [10, 27, 27])
    with pytest.raises(RuntimeError, match="position_ids"):
        ops.multimodal_rope_from_positions(q.transpose(1, 2).to(dev), k.transpose(1, 2).to(dev),
                                           pos[:, :, :5].to(dev), inv_freq, [16, 24, 24])


@pytest.mark.parametrize("layout", ["hf", "csrc"])
def test_mrope_from_packed_table_equals_the_positions_path(dev, layout):
    """multimodal_rope_from_table reads cos / sin from the packed table of multimodal_rope_table (256 bytes per token
    for the PyTorch path's layout, 512 for the CUDA kernel's, whose channels d and d + 64 take different planes; built
    once per forward); the table holds what the positions path evaluates per thread (the same device sincosf on
    the same angle, rounded to bf16), so forward and backward equal that path bit for bit -- at config 2's full size,
    through strided views, and for a short ragged sequence with distinct t / h / w positions -- and the oracle of the
    same layout within the stated tolerance."""
    ids, grid = wl.config2_tokens()
    pos, _ = oracle.rope_index_ref(ids, 2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, 2,
                                   image_grid_thw=grid)
    inv_freq = wl.text_inv_freq()
    q, k = wl.qk_inputs(16, 896)
    sec = list(wl.MROPE_SECTION)
    cases = [(q.transpose(1, 2), k.transpose(1, 2), pos)]  # [B, H, S, D] views of token-major memory
    q2, k2, pos2 = _pos_inputs(3, 37, torch.bfloat16, 31)
    cases.append((q2.transpose(1, 2).contiguous(), k2.transpose(1, 2).contiguous(), pos2))
    for qt, kt, p_ in cases:
        table = ops.multimodal_rope_table(p_.to(dev), inv_freq.to(dev), sec, layout)
        assert tuple(table.shape) == (p_.shape[1] * p_.shape[2], 64 if layout == "hf" else 128)
        qd, kd = qt.to(dev).requires_grad_(True), kt.to(dev).requires_grad_(True)
        tq, tk = ops.multimodal_rope_from_table(qd, kd, table, sec, layout)
        pq, pk = ops.multimodal_rope_from_positions(qt.to(dev), kt.to(dev), p_.to(dev), inv_freq.to(dev), sec, layout)
        assert _n_diff(tq.detach(), pq.cpu()) == 0 and _n_diff(tk.detach(), pk.cpu()) == 0
        cos, sin = oracle.rotary_cos_sin_ref(p_, inv_freq, torch.bfloat16)
        rq, rk = oracle.mrope_apply_ref(qt, kt, cos, sin, sec, layout)
        _close(tq.detach(), rq)
        _close(tk.detach(), rk)
        g = torch.Generator(device=dev).manual_seed(5)
        gq = torch.randn(tq.shape, device=dev, generator=g).to(torch.bfloat16)
        gk = torch.randn(tk.shape, device=dev, generator=g).to(torch.bfloat16)
        torch.autograd.backward([tq, tk], [gq, gk])
        bq, bk = torch.empty_like(gq), torch.empty_like(gk)
        native.rope_from_positions(gq, gk, p_.to(dev), inv_freq.to(dev), bq, bk, [2 * v for v in sec], backward=True,
                                   layout=layout)
        assert _n_diff(qd.grad, bq.cpu()) == 0 and _n_diff(kd.grad, bk.cpu()) == 0
    # what it cannot do is refused: fp16 (the table is bf16), a table built for the other layout (its width differs)
    table = ops.multimodal_rope_table(pos2.to(dev), inv_freq.to(dev), sec, layout)
    qh, kh = cases[1][0].to(dev), cases[1][1].to(dev)
    with pytest.raises(RuntimeError):
        native.rope_from_table(qh.half(), kh.half(), table, torch.empty_like(qh.half()), torch.empty_like(kh.half()),
                               [2 * v for v in sec], layout=layout)
    with pytest.raises(RuntimeError, match="same mrope_section and layout"):
        native.rope_from_table(qh, kh, table, torch.empty_like(qh), torch.empty_like(kh), [2 * v for v in sec],
                               layout="csrc" if layout == "hf" else "hf")


def test_extension_level_rope_uses_the_cuda_kernels_layout(dev):
    """wallx_csrc.rope / rope_bwd stand in for the reference's extension (csrc/ops.cu:11-21), whose kernel maps
    channels d < 32 -> t, d < 80 -> h, else w (csrc/rope.cu:104-117): called the way the reference's own ops.py
    calls them (ops.py:451-456, no layout argument) they must give that layout, not the PyTorch path's."""
    import wallx_csrc

    q, k, cos, sin = _inputs(2, 19, torch.bfloat16, 31)
    qt, kt = q.transpose(1, 2).contiguous(), k.transpose(1, 2).contiguous()
    doubled = [2 * s for s in wl.MROPE_SECTION]
    qo, ko = torch.empty_like(qt, device=dev), torch.empty_like(kt, device=dev)
    wallx_csrc.rope(qt.to(dev), kt.to(dev), cos.to(dev), sin.to(dev), qo, ko, doubled)
    rq, rk = oracle.mrope_apply_ref(qt, kt, cos, sin, list(wl.MROPE_SECTION), "csrc", eager_rounding=True)
    assert _n_diff(qo, rq) == 0 and _n_diff(ko, rk) == 0
    hq, _ = oracle.mrope_apply_ref(qt, kt, cos, sin, list(wl.MROPE_SECTION), "hf", eager_rounding=True)
    assert _n_diff(qo, hq) > 0
    g = torch.Generator().manual_seed(2)
    gq, gk = torch.randn(qt.shape, generator=g).to(torch.bfloat16), torch.randn(kt.shape, generator=g).to(torch.bfloat16)
    dq, dk = torch.empty_like(qo), torch.empty_like(ko)
    wallx_csrc.rope_bwd(gq.to(dev), gk.to(dev), qt.to(dev), kt.to(dev), cos.to(dev), sin.to(dev), dq, dk, doubled)
    bq, bk = oracle.mrope_apply_bwd_ref(gq, gk, cos, sin, list(wl.MROPE_SECTION), "csrc")
    _close(dq, bq)
    _close(dk, bk)
