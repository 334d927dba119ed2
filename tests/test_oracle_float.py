"""Pins the floating-point oracles (dual GEMM, SwiGLU FFN, M-RoPE, cos/sin builder)
against what the mathematics fixes.  CPU only."""

import math

import numpy as np
import pytest
import torch

import oracle
from wallx_mi355 import workloads as wl


# ----------------------------------------------------------------------------- GEMM / FFN
@pytest.mark.parametrize("trans_a,trans_b", [(False, False), (False, True), (True, False), (True, True)])
def test_dual_gemm_against_float64_contraction(trans_a, trans_b):
    g = torch.Generator().manual_seed(11)
    m0, m1, k0, k1, n0, n1 = 5, 3, 16, 8, 7, 4

    def mk(r, c, t):
        return torch.randn((c, r) if t else (r, c), generator=g).to(torch.bfloat16)

    a0, a1 = mk(m0, k0, trans_a), mk(m1, k1, trans_a)
    w0, w1 = mk(k0, n0, trans_b), mk(k1, n1, trans_b)
    o0, o1 = oracle.dual_gemm_ref(a0, a1, w0, w1, trans_a, trans_b)

    def f64(a, w):
        a, w = a.double().numpy(), w.double().numpy()
        a = a.T if trans_a else a
        w = w.T if trans_b else w
        return np.einsum("mk,kn->mn", a, w)

    for o, a, w in ((o0, a0, w0), (o1, a1, w1)):
        assert o.dtype == torch.bfloat16
        exact = torch.from_numpy(f64(a, w))
        # one bf16 rounding of an fp32 accumulation: relative error <= 2^-8 (+ fp32 noise)
        assert torch.all((o.double() - exact).abs() <= exact.abs() * 2 ** -8 + 1e-5)


def test_dual_gemm_empty_group():
    a0 = torch.zeros(0, 8, dtype=torch.bfloat16)
    a1 = torch.ones(2, 8, dtype=torch.bfloat16)
    w = torch.ones(3, 8, dtype=torch.bfloat16)
    o0, o1 = oracle.dual_gemm_ref(a0, a1, w, w, trans_b=True)
    assert o0.shape == (0, 3) and torch.equal(o1, torch.full((2, 3), 8.0, dtype=torch.bfloat16))


def test_swiglu_ffn_definition_fp32():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(6, 16, generator=g)
    gw, uw, dw = torch.randn(10, 16, generator=g), torch.randn(10, 16, generator=g), torch.randn(16, 10, generator=g)
    y = oracle.swiglu_ffn_ref(x, gw, uw, dw)
    gx = x.double() @ gw.double().T
    ref = ((gx / (1 + torch.exp(-gx))) * (x.double() @ uw.double().T)) @ dw.double().T
    assert torch.allclose(y.double(), ref, rtol=1e-5, atol=1e-5)
    # positively homogeneous of degree... no; but zero input gives zero output and down is linear:
    assert torch.equal(oracle.swiglu_ffn_ref(torch.zeros(2, 16), gw, uw, dw), torch.zeros(2, 16))
    y2 = oracle.swiglu_ffn_ref(x, gw, uw, 2 * dw)
    assert torch.allclose(y2, 2 * y, rtol=1e-6, atol=1e-6)


def test_swiglu_eager_rounding_close_to_fp32_math_in_bf16():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(32, 256, generator=g).to(torch.bfloat16)
    w = wl.expert_weights(256, 512, torch.bfloat16, g)
    a = oracle.swiglu_ffn_ref(x, *w.as_tuple(), eager_rounding=True).float()
    b = oracle.swiglu_ffn_ref(x, *w.as_tuple(), eager_rounding=False).float()
    assert torch.all((a - b).abs() <= 2e-2 + 1e-2 * b.abs())


def test_swiglu_bwd_against_central_differences_and_closed_forms():
    """dgate and dup of h = silu(g) * u: central differences of the float64 expression written out with exp (no
    library silu), silu'(0) = 1/2, silu'(x) -> 1 and silu(x) -> x for large x, -> 0 for very negative x."""
    g = torch.Generator().manual_seed(8)
    gate = torch.randn(64, 40, generator=g) * 2
    up = torch.randn(64, 40, generator=g)
    dh = torch.randn(64, 40, generator=g)
    hm, dg, du = oracle.swiglu_bwd_ref(gate, up, dh)
    G, U, D = gate.double().numpy(), up.double().numpy(), dh.double().numpy()
    h = lambda a, b: a / (1.0 + np.exp(-a)) * b
    eps = 1e-6
    num_dg = (h(G + eps, U) - h(G - eps, U)) / (2 * eps) * D
    num_du = (h(G, U + eps) - h(G, U - eps)) / (2 * eps) * D
    assert np.allclose(dg.double().numpy(), num_dg, rtol=1e-5, atol=1e-6)
    assert np.allclose(du.double().numpy(), num_du, rtol=1e-5, atol=1e-6)
    assert np.allclose(hm.double().numpy(), h(G, U), rtol=1e-5, atol=1e-6)
    one = torch.ones(4)
    _, dg0, du0 = oracle.swiglu_bwd_ref(torch.zeros(4), 3 * one, one)
    assert torch.allclose(dg0, 1.5 * one) and torch.all(du0 == 0)       # silu'(0) = 1/2, silu(0) = 0
    _, dgp, dup = oracle.swiglu_bwd_ref(30 * one, 2 * one, one)
    assert torch.allclose(dgp, 2 * one, atol=1e-6) and torch.allclose(dup, 30 * one, atol=1e-4)
    _, dgn, dun = oracle.swiglu_bwd_ref(-30 * one, 2 * one, one)
    assert torch.allclose(dgn, 0 * one, atol=1e-6) and torch.allclose(dun, 0 * one, atol=1e-6)
    # bf16: hmid carries the forward's rounding of silu before the product
    gb, ub = gate.to(torch.bfloat16), up.to(torch.bfloat16)
    hb, _, _ = oracle.swiglu_bwd_ref(gb, ub, dh.to(torch.bfloat16))
    want = (torch.nn.functional.silu(gb.float()).to(torch.bfloat16).float() * ub.float()).to(torch.bfloat16)
    assert torch.equal(hb, want)


def test_moe_block_matches_per_token_evaluation():
    """The block equals applying each token's own expert to that token alone."""
    g = torch.Generator().manual_seed(9)
    B, S, H = 2, 12, 32
    x = torch.randn(B, S, H, generator=g)
    types = torch.randint(0, 2, (B, S), generator=g) == 1
    ws = [wl.expert_weights(H, 48, torch.float32, g, 0.2), wl.expert_weights(H, 16, torch.float32, g, 0.2)]
    y = oracle.sparse_moe_block_ref(x, types, [w.as_tuple() for w in ws])
    for b in range(B):
        for s in range(S):
            e = int(types[b, s])
            ref = oracle.swiglu_ffn_ref(x[b, s:s + 1], *ws[e].as_tuple())
            assert torch.allclose(y[b, s], ref[0], rtol=1e-5, atol=1e-6)
    # an expert with no tokens contributes nothing and does not break the block
    y0 = oracle.sparse_moe_block_ref(x, torch.zeros(B, S, dtype=torch.bool), [w.as_tuple() for w in ws])
    assert torch.allclose(y0.view(-1, H), oracle.swiglu_ffn_ref(x.view(-1, H), *ws[0].as_tuple()), atol=1e-6)


def test_gated_ffn_with_other_activations_and_three_experts_against_a_scalar_loop():
    """`hidden_act` other than silu and an expert list of any length (act.py:71-77, 99-103, 142-154): the block
    against a float64 evaluation token by token, with gelu written through math.erf, the tanh form through math.tanh
    and relu through max -- nothing of the oracle's own expression is reused."""
    import math

    scalar = {
        "gelu": lambda v: 0.5 * v * (1.0 + math.erf(v / math.sqrt(2.0))),
        "gelu_pytorch_tanh": lambda v: 0.5 * v * (1.0 + math.tanh(math.sqrt(2.0 / math.pi) * (v + 0.044715 * v ** 3))),
        "relu": lambda v: max(v, 0.0),
        "silu": lambda v: v / (1.0 + math.exp(-v)),
    }
    g = torch.Generator().manual_seed(21)
    B, S, H = 2, 9, 8
    inters, acts = (6, 4, 10), ("gelu", "relu", "gelu_pytorch_tanh")
    x = torch.randn(B, S, H, generator=g)
    ids = torch.randint(0, 3, (B, S), generator=g)
    ws = [wl.expert_weights(H, i, torch.float32, g, 0.5).as_tuple() for i in inters]
    y = oracle.sparse_moe_block_ref(x, ids, ws, eager_rounding=False, acts=acts).double()
    for b in range(B):
        for s_ in range(S):
            e = int(ids[b, s_])
            gw, uw, dw = (t.double().tolist() for t in ws[e])
            xv = x[b, s_].double().tolist()
            hidden = []
            for i in range(inters[e]):
                gate = sum(a * w for a, w in zip(xv, gw[i]))
                up = sum(a * w for a, w in zip(xv, uw[i]))
                hidden.append(scalar[acts[e]](gate) * up)
            for o in range(H):
                want = sum(h * w for h, w in zip(hidden, dw[o]))
                assert abs(float(y[b, s_, o]) - want) <= 1e-5 + 1e-5 * abs(want), (b, s_, o)
    # the named functions themselves, on a grid of arguments
    t = torch.linspace(-6, 6, 49, dtype=torch.float64)
    for name, fn in scalar.items():
        got = oracle.activation_ref(name)(t)
        assert torch.allclose(got, torch.tensor([fn(float(v)) for v in t], dtype=torch.float64), rtol=1e-9, atol=1e-12)


# ----------------------------------------------------------------------------- M-RoPE
def _cos_sin(pos, dtype=torch.float32):
    return oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(), dtype)


def test_axis_maps():
    hf = oracle.mrope_axis_map(wl.MROPE_SECTION, 128, "hf").tolist()
    assert hf == [0] * 16 + [1] * 24 + [2] * 24 + [0] * 16 + [1] * 24 + [2] * 24
    cs = oracle.mrope_axis_map(wl.MROPE_SECTION, 128, "csrc").tolist()
    assert cs == [0] * 32 + [1] * 48 + [2] * 48
    assert sum(a != b for a, b in zip(hf, cs)) == 80
    assert all(hf[d] == hf[d + 64] for d in range(64))  # rotation pairs share an axis


def test_cos_sin_builder_closed_form():
    pos = torch.tensor([[[0, 1, 7]], [[0, 2, 9]], [[0, 3, 11]]])
    cos, sin = _cos_sin(pos)
    inv = wl.text_inv_freq()
    assert cos.shape == (3, 1, 3, 128)
    for a in range(3):
        for s in range(3):
            ang = pos[a, 0, s].float() * inv
            assert torch.equal(cos[a, 0, s, :64], torch.cos(ang)) and torch.equal(cos[a, 0, s, 64:], torch.cos(ang))
            assert torch.equal(sin[a, 0, s, :64], torch.sin(ang))
    assert math.isclose(float(inv[1]), 1e6 ** (-2 / 128), rel_tol=1e-6)


def test_mrope_reduces_to_textbook_rope_when_axes_agree():
    g = torch.Generator().manual_seed(1)
    B, S = 2, 5
    q = torch.randn(B, 4, S, 128, generator=g)
    k = torch.randn(B, 1, S, 128, generator=g)
    p = torch.randint(0, 50, (B, S), generator=g)
    pos = torch.stack([p, p, p])
    cos, sin = _cos_sin(pos)
    for layout in ("hf", "csrc"):
        qo, ko = oracle.mrope_apply_ref(q, k, cos, sin, list(wl.MROPE_SECTION), layout)
        ang = p[..., None].double() * wl.text_inv_freq().double()  # [B,S,64]
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        x1, x2 = q[..., :64].double(), q[..., 64:].double()
        ref = torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], -1)
        assert torch.allclose(qo.double(), ref, atol=1e-5)
    # position 0 is the identity
    z = torch.zeros(3, B, S, dtype=torch.long)
    cos0, sin0 = _cos_sin(z)
    qo, ko = oracle.mrope_apply_ref(q, k, cos0, sin0, list(wl.MROPE_SECTION))
    assert torch.equal(qo, q) and torch.equal(ko, k)


def test_mrope_hf_layout_is_a_rotation_per_pair_with_per_axis_angles():
    g = torch.Generator().manual_seed(8)
    B, S = 1, 6
    q = torch.randn(B, 2, S, 128, generator=g)
    k = torch.randn(B, 2, S, 128, generator=g)
    pos = torch.randint(0, 200, (3, B, S), generator=g)
    cos, sin = _cos_sin(pos)
    qo, _ = oracle.mrope_apply_ref(q, k, cos, sin, list(wl.MROPE_SECTION), "hf")
    n_in = q[..., :64] ** 2 + q[..., 64:] ** 2
    n_out = qo[..., :64] ** 2 + qo[..., 64:] ** 2
    assert torch.allclose(n_in, n_out, rtol=1e-4, atol=1e-5)
    # channel d rotates by pos[axis(d)] * inv_freq[d % 64]
    amap = oracle.mrope_axis_map(wl.MROPE_SECTION, 128, "hf")
    inv = wl.text_inv_freq().double()
    for d in (0, 15, 16, 39, 40, 63):
        ang = pos[amap[d], 0].double() * inv[d]  # [S]
        ref = q[0, 0, :, d].double() * torch.cos(ang) - q[0, 0, :, d + 64].double() * torch.sin(ang)
        assert torch.allclose(qo[0, 0, :, d].double(), ref, atol=1e-5)


def test_mrope_csrc_layout_per_channel_closed_form_with_distinct_axes():
    """The CUDA kernel's channel map (csrc/rope.cu:104-117: d < 32 -> t, d < 80 -> h, else w, thresholds from
    the elementwise-doubled sections [32, 48, 48]) with DIFFERENT t / h / w positions, channel by channel:
    out[d] = x[d] cos(p[axis(d)] f[d % 64]) -/+ x[d +/- 64] sin(p[axis(d)] f[d % 64]).  The two halves of a rotation
    pair take different planes here, so the hf layout, a swapped pair of planes or a shifted threshold all fail."""
    g = torch.Generator().manual_seed(18)
    B, S = 2, 5
    q = torch.randn(B, 3, S, 128, generator=g, dtype=torch.float64)
    k = torch.randn(B, 1, S, 128, generator=g, dtype=torch.float64)
    pos = torch.stack([torch.randint(0, 40, (B, S), generator=g), torch.randint(100, 140, (B, S), generator=g),
                       torch.randint(300, 340, (B, S), generator=g)])
    cos, sin = oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(), torch.float64)
    qo, ko = oracle.mrope_apply_ref(q, k, cos, sin, list(wl.MROPE_SECTION), "csrc")
    inv = wl.text_inv_freq().double()
    plane_of = lambda d: 0 if d < 32 else (1 if d < 80 else 2)  # noqa: E731  (written out from csrc/rope.cu:104-117)
    for x, xo in ((q, qo), (k, ko)):
        for d in range(128):
            ang = pos[plane_of(d)].double() * inv[d % 64]  # [B, S]
            if d < 64:
                ref = x[..., d] * torch.cos(ang)[:, None] - x[..., d + 64] * torch.sin(ang)[:, None]
            else:
                ref = x[..., d] * torch.cos(ang)[:, None] + x[..., d - 64] * torch.sin(ang)[:, None]
            assert torch.allclose(xo[..., d], ref, atol=2e-4), d  # the table builder forms the angle in fp32
    # and it is NOT the hf layout on these positions: the 80 channels whose plane differs all change
    qh, _ = oracle.mrope_apply_ref(q, k, cos, sin, list(wl.MROPE_SECTION), "hf")
    differs = [(qo[..., d] - qh[..., d]).abs().max() > 1e-7 for d in range(128)]
    hf_plane = [0] * 16 + [1] * 24 + [2] * 24
    assert [bool(v) for v in differs] == [plane_of(d) != hf_plane[d % 64] for d in range(128)]
    assert sum(bool(v) for v in differs) == 80


def test_mrope_against_transformers():
    try:
        from transformers.models.qwen2_5_vl.modeling_qwen2_5_vl import apply_multimodal_rotary_pos_emb as hf_apply
    except Exception:
        pytest.skip("transformers' qwen2_5_vl module is not importable")
    g = torch.Generator().manual_seed(21)
    q = torch.randn(2, 4, 7, 128, generator=g).to(torch.bfloat16)
    k = torch.randn(2, 2, 7, 128, generator=g).to(torch.bfloat16)
    pos = torch.randint(0, 300, (3, 2, 7), generator=g)
    cos, sin = _cos_sin(pos, torch.bfloat16)
    try:
        hq, hk = hf_apply(q, k, cos, sin, list(wl.MROPE_SECTION))
    except Exception as e:
        pytest.skip(f"signature drift: {e}")
    oq, ok = oracle.mrope_apply_ref(q, k, cos, sin, list(wl.MROPE_SECTION), "hf", eager_rounding=True)
    assert torch.equal(hq, oq) and torch.equal(hk, ok)


def test_mrope_backward_is_the_adjoint():
    g = torch.Generator().manual_seed(6)
    q = torch.randn(1, 2, 4, 128, generator=g, dtype=torch.float64)
    k = torch.randn(1, 1, 4, 128, generator=g, dtype=torch.float64)
    pos = torch.randint(0, 99, (3, 1, 4), generator=g)
    cos, sin = oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(), torch.float64)
    for layout in ("hf", "csrc"):
        qq = q.clone().requires_grad_(True)
        kk = k.clone().requires_grad_(True)
        qo, ko = oracle.mrope_apply_ref(qq, kk, cos, sin, list(wl.MROPE_SECTION), layout)
        gq, gk = torch.randn_like(qo), torch.randn_like(ko)
        (qo * gq).sum().backward(retain_graph=True)
        (ko * gk).sum().backward()
        bq, bk = oracle.mrope_apply_bwd_ref(gq, gk, cos, sin, list(wl.MROPE_SECTION), layout)
        assert torch.allclose(bq, qq.grad.to(bq.dtype), atol=1e-5)
        assert torch.allclose(bk, kk.grad.to(bk.dtype), atol=1e-5)


# ----------------------------------------------------------------------------- RMSNorm (caller fusion)
def test_rms_norm_against_library_routine_and_closed_form():
    g = torch.Generator().manual_seed(8)
    x = torch.randn(5, 33, 64, generator=g)
    w = torch.randn(64, generator=g)
    ref = torch.nn.functional.rms_norm(x, (64,), w, 1e-6)
    assert torch.allclose(oracle.rms_norm_ref(x, w, 1e-6), ref, rtol=1e-6, atol=1e-7)
    # a constant row c normalises to sign(c) (up to eps), so the output is sign(c) * weight
    c = torch.full((3, 64), -2.5)
    assert torch.allclose(oracle.rms_norm_ref(c, w, 0.0), -w.expand(3, 64), rtol=1e-6, atol=1e-7)
    # scaling the input leaves the output unchanged when eps = 0
    assert torch.allclose(oracle.rms_norm_ref(7.0 * x, w, 0.0), oracle.rms_norm_ref(x, w, 0.0), rtol=1e-5, atol=1e-6)
    # a dropped eps or a sum in place of the mean would fail this: one-hot row of magnitude a -> a / sqrt(a^2/n + eps)
    e = torch.zeros(1, 64); e[0, 3] = 0.01
    want = 0.01 / (0.01 ** 2 / 64 + 1e-3) ** 0.5
    assert abs(float(oracle.rms_norm_ref(e, torch.ones(64), 1e-3)[0, 3]) - want) < 1e-6


def test_rms_norm_against_transformers_module():
    try:
        from transformers.models.qwen2.modeling_qwen2 import Qwen2RMSNorm
    except Exception:
        pytest.skip("transformers' Qwen2RMSNorm is not importable")
    g = torch.Generator().manual_seed(9)
    x = torch.randn(4, 17, 128, generator=g).to(torch.bfloat16)
    m = Qwen2RMSNorm(128, eps=1e-6).to(torch.bfloat16)
    with torch.no_grad():
        m.weight.copy_(torch.randn(128, generator=g).to(torch.bfloat16))
        got = m(x)
    assert torch.equal(got, oracle.rms_norm_ref(x, m.weight.detach(), 1e-6))
