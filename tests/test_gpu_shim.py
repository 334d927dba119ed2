"""The nine names of the module that stands in for the reference's compiled extension (`wallx_csrc`, csrc/ops.cu:11-21),
each called with exactly the argument list of the reference's call site in wall_x/fusions/backend.py (positional, in
that order, the values ops.py prepares: int32-cast [T, K] ids with an empty workspace list, an empty CPU tensor for
absent probabilities, None for absent grids and mask, the doubled section list, an int32 grid) and compared with the
oracle.  The reference's own ops.py / backend.py cannot be imported here (their package needs CUDA-only and absent
dependencies), so this is the closest executable statement of "they run unchanged on this module"."""

import pytest
import torch

import oracle
import wallx_csrc
from wallx_mi355 import workloads as wl

pytestmark = pytest.mark.gpu


def _bf(shape, g, scale=1.0):
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


def test_asym_dual_gmm_as_backend_py_calls_it(dev):
    # backend.py:124-133: eight positional arguments, outputs allocated by the caller, both flags passed
    g = torch.Generator().manual_seed(1)
    in0, in1 = _bf((300, 256), g).to(dev), _bf((40, 128), g).to(dev)
    for trans_b in (False, True):
        w0 = _bf((512, 256) if trans_b else (256, 512), g, 0.05).to(dev)
        w1 = _bf((64, 128) if trans_b else (128, 64), g, 0.05).to(dev)
        out0 = torch.empty(300, 512, dtype=torch.bfloat16, device=dev)
        out1 = torch.empty(40, 64, dtype=torch.bfloat16, device=dev)
        assert wallx_csrc.asym_dual_gmm(in0, in1, w0, w1, out0, out1, False, trans_b) is None
        r0, r1 = oracle.dual_gemm_ref(in0.cpu(), in1.cpu(), w0.cpu(), w1.cpu(), False, trans_b)
        for got, ref in ((out0, r0), (out1, r1)):
            err = (got.float().cpu() - ref.float()).abs()
            assert bool((err <= 2e-2 + 1e-2 * ref.float().abs()).all())


def test_permute_unpermute_as_ops_py_calls_them(dev):
    g = torch.Generator().manual_seed(2)
    T, K, H = 700, 2, 64
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    ids = torch.randint(0, 5, (T, K), generator=g)
    # ops.py:219-224, 245-251: ids cast to int32, [T, K]; the class-level workspace starts as an empty list and the
    # returned one is passed back on the next call; max_expanded_token_num = T * K
    ids32 = ids.to(torch.int32).to(dev)
    workspace = []
    permuted, row_id_map, workspace = wallx_csrc.permute(x.to(dev), ids32, 0, workspace, T * K)
    ref_p, ref_map, _ = oracle.permute_ref(x, ids)
    assert row_id_map.dtype == torch.int32 and torch.equal(row_id_map.cpu(), ref_map)
    assert torch.equal(permuted.cpu(), ref_p)
    again, map2, workspace2 = wallx_csrc.permute(x.to(dev), ids32, 0, workspace, T * K)
    assert torch.equal(again, permuted) and torch.equal(map2, row_id_map) and isinstance(workspace2, list)
    # ops.py:353-359: probabilities fp32 [T, K]; backend.py:197
    probs = torch.rand(T, K, generator=g)
    out = wallx_csrc.unpermute(permuted, row_id_map, probs.to(dev), T, K)
    assert torch.equal(out.cpu(), oracle.unpermute_ref(ref_p, ref_map, probs))
    # ops.py:271-273 (backward of permute): no probabilities = an empty CPU tensor, topK of the forward
    ids1 = ids[:, :1].contiguous()
    p1, m1, _ = wallx_csrc.permute(x.to(dev), ids1.to(torch.int32).to(dev), 0, [], T)
    out1 = wallx_csrc.unpermute(p1, m1, torch.tensor([]), T, 1)
    assert torch.equal(out1.cpu(), x)  # permute then unpermute at K = 1 is the identity
    # ops.py:377-379 / backend.py:230: (act_grad, prob_grad) of the weighted combine
    grad = torch.randn(T, H, generator=g).to(torch.bfloat16)
    act_grad, prob_grad = wallx_csrc.unpermute_bwd(grad.to(dev), permuted, row_id_map, probs.to(dev))
    ra, rp, _ = oracle.unpermute_bwd_ref(grad, ref_p, ref_map, probs)
    assert torch.equal(act_grad.cpu(), ra)
    assert prob_grad.dtype == torch.float32 and torch.allclose(prob_grad.cpu(), rp, rtol=1e-5, atol=1e-4)


def test_rope_and_rope_bwd_as_ops_py_calls_them(dev):
    # ops.py:451-456: the section list doubled element by element, contiguous [B, H, S, D] q / k, outputs allocated by
    # the caller; no layout argument exists in the reference, so the module gives the CUDA kernel's channel layout
    g = torch.Generator().manual_seed(3)
    B, S, D = 2, 45, 128
    q, k = _bf((B, 16, S, D), g), _bf((B, 2, S, D), g)
    pos = torch.stack([torch.randint(0, 50, (B, S), generator=g), torch.randint(60, 90, (B, S), generator=g),
                       torch.randint(100, 150, (B, S), generator=g)])
    cos, sin = oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(), torch.bfloat16)
    doubled = [s * 2 for s in wl.MROPE_SECTION]
    q_out, k_out = torch.empty_like(q, device=dev), torch.empty_like(k, device=dev)
    assert wallx_csrc.rope(q.to(dev), k.to(dev), cos.to(dev), sin.to(dev), q_out, k_out, doubled) is None
    rq, rk = oracle.mrope_apply_ref(q, k, cos, sin, list(wl.MROPE_SECTION), "csrc", eager_rounding=True)
    assert torch.equal(q_out.cpu(), rq) and torch.equal(k_out.cpu(), rk)
    # ops.py:481-491: nine positional arguments
    gq, gk = _bf(tuple(q.shape), g), _bf(tuple(k.shape), g)
    dq, dk = torch.empty_like(q_out), torch.empty_like(k_out)
    assert wallx_csrc.rope_bwd(gq.to(dev), gk.to(dev), q.to(dev), k.to(dev), cos.to(dev), sin.to(dev), dq, dk,
                               doubled) is None
    bq, bk = oracle.mrope_apply_bwd_ref(gq, gk, cos, sin, list(wl.MROPE_SECTION), "csrc")
    for got, ref in ((dq, bq), (dk, bk)):
        err = (got.float().cpu() - ref.float()).abs()
        assert bool((err <= 2e-2 + 1e-2 * ref.float().abs()).all())


def test_index_builders_as_backend_py_calls_them(dev):
    ids, grid = wl.config2_tokens(batch=3)
    args = (2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID)
    # backend.py:341-352: ten positional arguments, None for the absent video grid, intervals and mask
    pos, deltas = wallx_csrc.rope_index(ids.to(dev), grid.to(dev), None, None, None, *args, 2.0)
    rpos, rdeltas = oracle.rope_index_ref(ids, *args, 2.0, image_grid_thw=grid)
    assert pos.dtype == torch.int64 and torch.equal(pos.cpu(), rpos) and torch.equal(deltas.cpu(), rdeltas)
    # text only, with a mask: both grids None
    text = torch.randint(1000, 2000, (2, 17))
    mask = torch.ones(2, 17, dtype=torch.int64)
    mask[0, :5] = 0
    tpos, tdel = wallx_csrc.rope_index(text.to(dev), None, None, None, mask.to(dev), *args, 2.0)
    rtpos, rtdel = oracle.rope_index_ref(text, *args, 2.0, attention_mask=mask)
    assert torch.equal(tpos.cpu(), rtpos) and torch.equal(tdel.cpu(), rtdel)
    # backend.py:387: three positional arguments
    inv = wl.vision_inv_freq()
    table = wallx_csrc.rot_pos_emb(inv.to(dev), grid.to(dev), 2)
    assert torch.equal(table.cpu(), oracle.rot_pos_emb_ref(inv, grid, 2))
    # backend.py:427-433: five positional arguments, the grid cast to int32 and the window size already divided
    # (ops.py:723-740)
    wi, cu = wallx_csrc.get_window_index(grid.to(torch.int32).to(dev), 2, 112 // 2 // 14, 14, 4)
    rwi, rcu = oracle.window_index_dedup_ref(grid, 112, 2, 14, 4)
    assert wi.dtype == torch.int32 and torch.equal(wi.cpu(), rwi) and torch.equal(cu.cpu(), rcu)
