"""The prefill harness (config 5's decoder shape, shrunk) against a plain forward of the same weights built from the
oracle's pieces on the CPU in fp32: positions from rope_index_ref, M-RoPE from mrope_apply_ref, the dual-expert
block from sparse_moe_block_ref, attention written out as softmax(QK^T)V with the stated mask."""

import math

import pytest
import torch

import oracle
from wallx_mi355 import workloads as wl

pytestmark = pytest.mark.gpu


def _ref_forward(h, ids, grid, types, mask_mode):
    B, S = ids.shape
    D, nq, nkv, eps = h.head_dim, h.n_q, h.n_kv, h.eps
    f = lambda t: t.float().cpu()

    def norm(x, w):
        return f(w) * (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps))

    pos, _ = oracle.rope_index_ref(ids.cpu(), 2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, 2,
                                   image_grid_thw=grid.cpu())
    cos, sin = oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(D), torch.bfloat16)
    cos, sin = cos.float(), sin.float()
    allow = torch.ones(S, S, dtype=torch.bool).tril()[None, None].expand(B, 1, S, S)
    if mask_mode == "action_block":
        t = types.cpu()
        allow = allow | (t[:, None, :, None] & t[:, None, None, :])
    x = f(h.embed)[ids.cpu()]
    for layer in h.layers:
        qkv = norm(x, layer["ln1"]) @ f(layer["wqkv"]).T + f(layer["bqkv"])
        q, k, v = qkv.split([nq * D, nkv * D, nkv * D], dim=-1)
        q = q.view(B, S, nq, D).transpose(1, 2)
        k = k.view(B, S, nkv, D).transpose(1, 2)
        v = v.view(B, S, nkv, D).transpose(1, 2)
        q, k = oracle.mrope_apply_ref(q, k, cos, sin, list(wl.MROPE_SECTION), eager_rounding=False)
        k, v = k.repeat_interleave(nq // nkv, 1), v.repeat_interleave(nq // nkv, 1)
        s = (q @ k.transpose(-1, -2)) / math.sqrt(D)
        a = torch.softmax(s.masked_fill(~allow, float("-inf")), -1) @ v
        x = x + a.transpose(1, 2).reshape(B, S, nq * D) @ f(layer["wo"]).T
        ws = [tuple(f(w) for w in e) for e in layer["experts"]]
        x = x + oracle.sparse_moe_block_ref(norm(x, layer["ln2"]), types.cpu(), ws, eager_rounding=False)
    return norm(x[:, -1], h.final_ln) @ f(h.embed).T


@pytest.mark.parametrize("mask_mode,fuse,suffix,qkv", [("causal", True, None, False), ("action_block", True, None, False),
                                                      ("action_block", True, 8, False), ("causal", False, None, False),
                                                      ("action_block", True, 8, True)])
def test_prefill_harness_matches_plain_forward(dev, mask_mode, fuse, suffix, qkv):
    from wallx_mi355 import harness

    h = harness.PrefillHarness(n_layers=2, hidden=256, n_q=4, n_kv=2, head_dim=128, inter=(512, 256), vocab=151936,
                               device=dev, seed=3, mask=mask_mode, keep_dense=True, fuse=fuse, fuse_qkv_rope=qkv,
                               o_proj_native=qkv)
    row = wl.vla_row_tokens(n_images=1, image_tokens=16, lead_text=5, tail_text=9, n_action=8)
    ids = torch.tensor([row, row, row], dtype=torch.int64, device=dev)
    grid = torch.tensor([[1, 8, 8]] * 3, dtype=torch.int64, device=dev)
    types = ids == wl.ACTION_TOKEN_ID
    timer = harness.OpTimer()
    got = h.forward(ids, grid, types, timer, action_suffix=suffix).float().cpu()
    split = timer.report_ms()
    movers = {"rmsnorm+permute", "unpermute+residual+rmsnorm"} if fuse else {"permute", "unpermute"}
    assert movers | {"ffn_gate_up_swiglu", "ffn_down", "qkv_proj+mrope" if qkv else "mrope", "rope_index", "sdpa_torch"} <= set(split)
    ref = _ref_forward(h, ids, grid, types, mask_mode)
    # bf16 storage of every intermediate over two layers against an fp32 forward: bound the error by the logits' scale
    scale = float(ref.abs().max())
    err = float((got - ref).abs().max())
    assert err <= 0.04 * scale, f"max |diff| {err} vs logits scale {scale}"


def test_config5_full_shape_piece_by_piece(dev):
    """Config 5 at its stated shape (36 layers, hidden 2048, 16 query / 2 KV heads of 128, experts 11008 / 1024,
    16 sequences x 912 tokens, bf16 N(0, 0.02)).  A CPU forward of the whole model is out of reach, so the forward
    is checked piece by piece on what the kernels actually read and wrote inside it: the position ids exactly, and
    for layers 0 / 17 / 35 the M-RoPE output and the layer's closing half (RMSNorm -> permute -> both experts' FFN
    -> unpermute -> residual -> next RMSNorm) on sampled tokens, each against the oracle on the captured input."""
    from wallx_mi355 import harness

    layers = (0, 17, 35)
    h = harness.PrefillHarness(device=dev, seed=0, mask="action_block", keep_dense=layers)
    assert (h.n_layers, h.hidden, h.n_q, h.n_kv, h.head_dim, tuple(h.inter)) == (36, 2048, 16, 2, 128, (11008, 1024))
    ids, grid, types = harness.config5_inputs(16, dev)
    assert ids.shape == (16, 912) and int(types.sum()) == 16 * 32
    cap = {"layers": layers}
    logits = h.forward(ids, grid, types, action_suffix=32, capture=cap)
    assert logits.shape == (16, 151936) and bool(torch.isfinite(logits.float()).all())
    # position ids: bit-exact
    rpos, _ = oracle.rope_index_ref(ids.cpu(), 2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, 2,
                                    image_grid_thw=grid.cpu())
    assert torch.equal(cap["pos"].cpu(), rpos)
    cos, sin = oracle.rotary_cos_sin_ref(rpos, wl.text_inv_freq(128), torch.bfloat16)
    tf = types.view(-1).cpu()
    g = torch.Generator().manual_seed(5)
    T = tf.numel()
    act, vl = torch.nonzero(tf).flatten(), torch.nonzero(~tf).flatten()
    pick = torch.cat([vl[torch.randperm(vl.numel(), generator=g)[:40]], vl[:2], vl[-2:],
                      act[torch.randperm(act.numel(), generator=g)[:12]], act[:2], act[-2:]])
    for li in layers:
        c = cap[li]
        # M-RoPE inside the forward (cos / sin evaluated on the device from the position ids): two batch rows in full.
        # With the rotation in the projection's epilogue (the default) q and k before the rotation exist nowhere on
        # the device: the oracle projects the captured layer input with the layer's weights itself.
        for b in (0, 15):
            if "q_in" in c:
                q_in, k_in = c["q_in"][b:b + 1].cpu(), c["k_in"][b:b + 1].cpu()
            else:
                lay = h.layers[li]
                qkv = torch.nn.functional.linear(c["x_in"][b].float().cpu(), lay["wqkv"].float().cpu(),
                                                 lay["bqkv"].float().cpu()).to(torch.bfloat16)
                q_in = qkv[:, :h.n_q * 128].reshape(1, -1, h.n_q, 128).transpose(1, 2)
                k_in = qkv[:, h.n_q * 128:(h.n_q + h.n_kv) * 128].reshape(1, -1, h.n_kv, 128).transpose(1, 2)
            rq, rk = oracle.mrope_apply_ref(q_in, k_in, cos[:, b:b + 1], sin[:, b:b + 1], list(wl.MROPE_SECTION))
            for got, ref, what in ((c["q_out"][b:b + 1], rq, "q"), (c["k_out"][b:b + 1], rk, "k")):
                err = (got.float().cpu() - ref.float()).abs()
                assert bool((err <= 2e-2 + 1e-2 * ref.float().abs()).all()), f"layer {li} M-RoPE {what}: {float(err.max())}"
                # the device's sincosf against the CPU table builder's: a bf16 step on a small share of the entries
                assert float((got.cpu() != ref).float().mean()) < 5e-3
        # closing half of the layer on sampled tokens
        layer = h.layers[li]
        hin = c["ffn_in"][pick.to(dev)].cpu()
        ws = [tuple(w.cpu() for w in e) for e in layer["experts"]]
        xn = oracle.rms_norm_ref(hin, layer["ln2"].cpu(), h.eps)
        y = oracle.sparse_moe_block_ref(xn[None], tf[pick][None], ws)[0]
        ref_out = (hin.float() + y.float()).to(torch.bfloat16)
        got_out = c["ffn_out"].view(T, -1)[pick.to(dev)].cpu()
        err = (got_out.float() - ref_out.float()).abs()
        assert bool((err <= 2e-2 + 1e-2 * ref_out.float().abs()).all()), f"layer {li} FFN + residual: {float(err.max())}"
        nxt = h.layers[li + 1]["ln1"] if li + 1 < h.n_layers else h.final_ln
        ref_n = oracle.rms_norm_ref(got_out, nxt.cpu(), h.eps)  # the norm of what the kernel itself stored
        got_n = c["next_normed"].view(T, -1)[pick.to(dev)].cpu()
        err = (got_n.float() - ref_n.float()).abs()
        assert bool((err <= 2e-2 + 1e-2 * ref_n.float().abs()).all()), f"layer {li} next RMSNorm: {float(err.max())}"
