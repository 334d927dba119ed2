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


@pytest.mark.parametrize("mask_mode,fuse,suffix", [("causal", True, None), ("action_block", True, None),
                                                  ("action_block", True, 8), ("causal", False, None)])
def test_prefill_harness_matches_plain_forward(dev, mask_mode, fuse, suffix):
    from wallx_mi355 import harness

    h = harness.PrefillHarness(n_layers=2, hidden=256, n_q=4, n_kv=2, head_dim=128, inter=(512, 256), vocab=151936,
                               device=dev, seed=3, mask=mask_mode, keep_dense=True, fuse=fuse)
    row = wl.vla_row_tokens(n_images=1, image_tokens=16, lead_text=5, tail_text=9, n_action=8)
    ids = torch.tensor([row, row, row], dtype=torch.int64, device=dev)
    grid = torch.tensor([[1, 8, 8]] * 3, dtype=torch.int64, device=dev)
    types = ids == wl.ACTION_TOKEN_ID
    timer = harness.OpTimer()
    got = h.forward(ids, grid, types, timer, action_suffix=suffix).float().cpu()
    split = timer.report_ms()
    movers = {"rmsnorm+permute", "unpermute+residual+rmsnorm"} if fuse else {"permute", "unpermute"}
    assert movers | {"ffn_gate_up_swiglu", "ffn_down", "mrope", "rope_index", "sdpa_torch"} <= set(split)
    ref = _ref_forward(h, ids, grid, types, mask_mode)
    # bf16 storage of every intermediate over two layers against an fp32 forward: bound the error by the logits' scale
    scale = float(ref.abs().max())
    err = float((got - ref).abs().max())
    assert err <= 0.04 * scale, f"max |diff| {err} vs logits scale {scale}"
