"""Pins the integer oracles (permute, rope_index, rot_pos, window_index) against
independent facts: brute force, closed forms, the reference's docstring vector,
and transformers' same-lineage functions where they import.  CPU only."""

import itertools

import numpy as np
import pytest
import torch

import oracle
from wallx_mi355 import workloads as wl


# ----------------------------------------------------------------------------- permute
def _brute_partition(ids_2d):
    """Stable partition by definition: walk experts in increasing order, rows in order."""
    T, K = ids_2d.shape
    flat = ids_2d.reshape(-1).tolist()
    order = []
    for e in sorted(set(flat)):
        order += [i for i, v in enumerate(flat) if v == e]
    return order  # position -> flat row id


@pytest.mark.parametrize("T,E,K", [(1, 1, 1), (7, 2, 1), (64, 4, 1), (33, 3, 2), (16, 4, 2)])
def test_permute_bruteforce(T, E, K):
    g = torch.Generator().manual_seed(T * 100 + E * 10 + K)
    ids = torch.randint(0, E, (T, K), generator=g, dtype=torch.int32)
    x = torch.randn(T, 8, generator=g)
    permuted, rmap, srt = oracle.permute_ref(x, ids if K > 1 else ids[:, 0])
    order = _brute_partition(ids.numpy())
    assert srt.tolist() == order
    for p, src in enumerate(order):
        t, k = divmod(src, K)
        assert rmap[k * T + t].item() == p
        assert torch.equal(permuted[p], x[t])
    assert sorted(rmap.tolist()) == list(range(T * K))


def test_permute_num_out_tokens_drops_tail():
    ids = torch.tensor([1, 0, 1, 0, 0, 1], dtype=torch.int32)
    x = torch.arange(6, dtype=torch.float32)[:, None].repeat(1, 4)
    permuted, rmap, _ = oracle.permute_ref(x, ids, num_out_tokens=4)
    assert permuted.shape[0] == 4
    assert permuted[:, 0].tolist() == [1, 3, 4, 0]
    assert rmap.tolist() == [3, 0, -1, 1, 2, -1]
    y = oracle.unpermute_ref(permuted, rmap)
    assert y[:, 0].tolist() == [0, 1, 0, 3, 4, 0]  # dropped rows come back as zeros


def test_permute_roundtrip_and_config1_identity():
    x, types, _ = wl.config1()
    xf = x.view(-1, x.shape[-1])
    permuted, rmap, _ = oracle.permute_ref(xf, types.view(-1))
    assert torch.equal(rmap, torch.arange(512, dtype=torch.int32))  # tail mask => identity
    assert torch.equal(permuted, xf)
    g = torch.Generator().manual_seed(3)
    ids = torch.randint(0, 2, (1000,), generator=g) == 1
    xb = torch.randn(1000, 16, generator=g).to(torch.bfloat16)
    p, m, _ = oracle.permute_ref(xb, ids)
    assert torch.equal(oracle.unpermute_ref(p, m), xb)
    off = oracle.expert_offsets_ref(ids, 2)
    assert off.tolist() == [0, int((~ids).sum()), 1000]
    assert torch.equal(p[: off[1]], xb[~ids]) and torch.equal(p[off[1]:], xb[ids])


def test_unpermute_topk2_weighted_sum_fp32():
    g = torch.Generator().manual_seed(5)
    T, K, H = 9, 2, 4
    ids = torch.randint(0, 3, (T, K), generator=g, dtype=torch.int32)
    x = torch.randn(T, H, generator=g)
    p, rmap, _ = oracle.permute_ref(x, ids)
    probs = torch.rand(T, K, generator=g)
    y = oracle.unpermute_ref(p, rmap, probs)
    # every expert copy of token t is x[t], so the result is x[t] * sum_k prob[t, k]
    assert torch.allclose(y, x * probs[:, :1] + x * probs[:, 1:], rtol=0, atol=1e-6)
    # K == 1 ignores probabilities entirely (csrc/permute.cu:405-415)
    p1, m1, _ = oracle.permute_ref(x, ids[:, 0])
    assert torch.equal(oracle.unpermute_ref(p1, m1, torch.rand(T, 1, generator=g)), x)


def _scalar_unpermute(y, rmap, probs, T, K):
    """out[t] = sum_k p[t, k] * y[map[k*T + t]] written as scalar loops over differentiable tensors."""
    rows = []
    for t in range(T):
        acc = torch.zeros(y.shape[1], dtype=y.dtype)
        for k in range(K):
            r = int(rmap[k * T + t])
            if r >= 0:
                acc = acc + (probs[t, k] * y[r] if K > 1 else y[r])
        rows.append(acc)
    return torch.stack(rows)


@pytest.mark.parametrize("T,E,K,drop", [(1, 1, 1, 0), (8, 2, 1, 0), (8, 2, 1, 3), (7, 3, 2, 0), (6, 4, 3, 5), (5, 2, 2, 4)])
def test_unpermute_bwd_is_the_autograd_gradient(T, E, K, drop):
    """unpermute_bwd_ref against torch autograd of the fp32 expression it is the backward of, on tiny inputs
    (with and without rows dropped by num_out_tokens).  A transposed map index, a missing probability factor on
    act_grad, or a prob_grad taken against the wrong row each fail this."""
    g = torch.Generator().manual_seed(1000 * T + 100 * E + 10 * K + drop)
    H = 5
    ids = torch.randint(0, E, (T, K), generator=g, dtype=torch.int32)
    n_out = T * K - drop
    x = torch.randn(T, H, generator=g)
    permuted, rmap, _ = oracle.permute_ref(x, ids if K > 1 else ids[:, 0], num_out_tokens=n_out if drop else 0)
    y = torch.randn(permuted.shape[0], H, generator=g).requires_grad_(True)  # any sorted-space activations
    probs = torch.rand(T, K, generator=g).requires_grad_(True)
    out = _scalar_unpermute(y, rmap, probs, T, K)
    # the forward oracle is the same function
    assert torch.allclose(oracle.unpermute_ref(y.detach(), rmap, probs.detach(), T, K), out.detach(), atol=1e-6)
    grad_out = torch.randn(T, H, generator=g)
    (out * grad_out).sum().backward()
    act_grad, prob_grad, written = oracle.unpermute_bwd_ref(grad_out, y.detach(), rmap, probs.detach())
    assert torch.allclose(act_grad, y.grad, atol=1e-6)
    # rows no token maps to: the oracle reports them as unwritten (their gradient is zero)
    mapped = torch.zeros(permuted.shape[0], dtype=torch.bool)
    mapped[rmap[rmap >= 0].long()] = True
    assert torch.equal(written, mapped) and bool((y.grad[~mapped] == 0).all())
    if K > 1:
        assert torch.allclose(prob_grad, probs.grad, atol=1e-5)
    else:
        assert float(prob_grad.abs().max()) == 0.0  # csrc/permute.cu:405-415: probabilities play no part at K == 1


def test_unpermute_bwd_is_the_adjoint_of_unpermute():
    """<unpermute(y), g> == <y, unpermute_bwd(g)> for fixed probabilities (fp64-exact inputs in fp32)."""
    g = torch.Generator().manual_seed(77)
    T, K, H = 11, 2, 6
    ids = torch.randint(0, 3, (T, K), generator=g, dtype=torch.int32)
    _, rmap, _ = oracle.permute_ref(torch.zeros(T, H), ids)
    y = torch.randint(-8, 8, (T * K, H), generator=g).float()
    go = torch.randint(-8, 8, (T, H), generator=g).float()
    probs = torch.randint(0, 4, (T, K), generator=g).float() / 4  # exact in every dtype
    lhs = (oracle.unpermute_ref(y, rmap, probs) * go).sum()
    act_grad, _, _ = oracle.unpermute_bwd_ref(go, y, rmap, probs)
    assert float(lhs) == float((y * act_grad).sum())


def test_unpermute_topk_bf16_exact_cases_and_rounding_bound():
    """bf16 at topK > 1.  Where every product and partial sum is representable the result is the exact one,
    whatever the rounding order; in general it stays within K roundings of the fp32 value."""
    g = torch.Generator().manual_seed(12)
    T, K, H = 16, 3, 8
    ids = torch.stack([torch.randperm(4, generator=g)[:K] for _ in range(T)]).to(torch.int32)
    x = torch.randint(-16, 16, (T, H), generator=g).to(torch.bfloat16)        # small integers
    probs = (2.0 ** -torch.randint(0, 3, (T, K), generator=g).float())          # powers of two
    p, rmap, _ = oracle.permute_ref(x, ids)
    got = oracle.unpermute_ref(p, rmap, probs)
    assert got.dtype == torch.bfloat16
    assert torch.equal(got.double(), x.double() * probs.double().sum(1, keepdim=True))
    # general values: each of the K products and K - 1 sums rounds once (relative 2^-9 each)
    xr = torch.randn(T, H, generator=g).to(torch.bfloat16)
    pr = torch.rand(T, K, generator=g)
    p, rmap, _ = oracle.permute_ref(xr, ids)
    got = oracle.unpermute_ref(p, rmap, pr).double()
    exact = xr.double() * pr.to(torch.bfloat16).double().sum(1, keepdim=True)
    bound = (2 * K) * 2.0 ** -9 * (xr.double().abs() * pr.double().sum(1, keepdim=True)) + 1e-30
    assert bool(((got - exact).abs() <= bound).all())


# ----------------------------------------------------------------------------- rope_index
def test_rope_index_reference_docstring_vector():
    """vl.py:1744-1760: a 3x2x2 (after merge) video at 2 temporal patches per second with
    tokens_per_second = 25 followed by five text tokens."""
    V, TXT = wl.VIDEO_TOKEN_ID, wl.TEXT_TOKEN_ID
    ids = torch.tensor([[wl.VISION_START_TOKEN_ID] + [V] * 12 + [TXT] * 5])
    # merge 2 -> pre-merge grid (3, 4, 4); interval = 25 * 2s... the docstring uses
    # tokens_per_second 25 and second_per_grid 2.0 -> temporal ids 0, 50, 100
    pos, delta = oracle.rope_index_ref(
        ids, 2, wl.IMAGE_TOKEN_ID, V, wl.VISION_START_TOKEN_ID, 25,
        video_grid_thw=torch.tensor([[3, 4, 4]]), second_per_grid_ts=torch.tensor([2.0]))
    # the leading <vision_start> takes position 0, so the documented vectors appear shifted by 1
    vis = pos[:, 0, 1:13] - 1
    assert vis[0].tolist() == [0, 0, 0, 0, 50, 50, 50, 50, 100, 100, 100, 100]
    assert vis[1].tolist() == [0, 0, 1, 1, 0, 0, 1, 1, 0, 0, 1, 1]
    assert vis[2].tolist() == [0, 1, 0, 1, 0, 1, 0, 1, 0, 1, 0, 1]
    # text resumes at max(vision) + 1 = 101 (+1 shift), all three axes equal
    txt = pos[:, 0, 13:] - 1
    assert txt[0].tolist() == [101, 102, 103, 104, 105]
    assert torch.equal(txt[0], txt[1]) and torch.equal(txt[0], txt[2])
    assert delta.tolist() == [[107 - 18]]


def test_rope_index_config2_closed_form():
    ids, grid = wl.config2_tokens()
    pos, delta = oracle.rope_index_ref(ids, 2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID,
                                       wl.VISION_START_TOKEN_ID, 2, image_grid_thw=grid)
    assert pos.shape == (3, 16, 896) and pos.dtype == torch.int64
    assert int(pos.max()) == 175
    assert delta.tolist() == [[-720]] * 16
    # closed form for one row, written independently of the oracle's walk
    exp = np.zeros((3, 896), dtype=np.int64)
    cur, i = 0, 0
    exp[:, :11] = np.arange(11)
    i, cur = 11, 11
    for img in range(3):
        hh, ww = np.divmod(np.arange(256), 16)
        exp[0, i:i + 256] = cur
        exp[1, i:i + 256] = cur + hh
        exp[2, i:i + 256] = cur + ww
        i += 256
        cur += 16
        n_text = 2 if img < 2 else 1 + 80 + 32
        exp[:, i:i + n_text] = cur + np.arange(n_text)
        i += n_text
        cur += n_text
    assert i == 896
    for b in range(16):
        assert np.array_equal(pos[:, b].numpy(), exp)


def test_rope_index_text_only_and_padding():
    ids = torch.full((2, 6), wl.TEXT_TOKEN_ID)
    mask = torch.tensor([[0, 0, 1, 1, 1, 1], [1, 1, 1, 1, 1, 1]])
    pos, delta = oracle.rope_index_ref(ids, 2, 1, 2, 3, 2, attention_mask=mask)
    assert pos[0].tolist() == [[1, 1, 0, 1, 2, 3], [0, 1, 2, 3, 4, 5]]
    assert delta.tolist() == [[-2], [0]]
    pos, delta = oracle.rope_index_ref(ids, 2, 1, 2, 3, 2)
    assert pos[2, 1].tolist() == list(range(6)) and delta.tolist() == [[0], [0]]
    # left padding with an image: valid tokens are numbered as if the pads were absent
    row = [wl.TEXT_TOKEN_ID] * 3 + [wl.VISION_START_TOKEN_ID] + [wl.IMAGE_TOKEN_ID] * 4 + [wl.TEXT_TOKEN_ID]
    ids = torch.tensor([row])
    mask = torch.tensor([[0, 0, 1] + [1] * 6])
    pos, delta = oracle.rope_index_ref(ids, 2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID,
                                       wl.VISION_START_TOKEN_ID, 2,
                                       image_grid_thw=torch.tensor([[1, 4, 4]]), attention_mask=mask)
    assert pos[0, 0].tolist() == [1, 1, 0, 1, 2, 2, 2, 2, 4]
    assert pos[1, 0].tolist() == [1, 1, 0, 1, 2, 2, 3, 3, 4]
    assert pos[2, 0].tolist() == [1, 1, 0, 1, 2, 3, 2, 3, 4]
    assert delta.tolist() == [[5 - 9]]


def test_rope_index_grid_cursor_runs_across_rows_and_mixed_media():
    I, V, S0, T = wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, wl.TEXT_TOKEN_ID
    # row 0: video(2 frames of 1x2) then image(2x1); row 1: image(1x1) only, padded on the right
    r0 = [S0] + [V] * 4 + [T] + [S0] + [I] * 2 + [T]
    r1 = [T, S0, I, T] + [T] * 6
    ids = torch.tensor([r0, r1])
    mask = torch.tensor([[1] * 10, [1] * 4 + [0] * 6])
    pos, delta = oracle.rope_index_ref(
        ids, 2, I, V, S0, 2.0,
        image_grid_thw=torch.tensor([[1, 4, 2], [1, 2, 2]]),
        video_grid_thw=torch.tensor([[2, 2, 4]]),
        second_per_grid_ts=torch.tensor([1.5]), attention_mask=mask)
    # video: t ids trunc(t * 1.5 * 2.0) = 0, 3 ; w ids 0, 1
    assert pos[0, 0].tolist() == [0, 1, 1, 4, 4, 5, 6, 7, 7, 9]
    assert pos[1, 0].tolist() == [0, 1, 1, 1, 1, 5, 6, 7, 8, 9]
    assert pos[2, 0].tolist() == [0, 1, 2, 1, 2, 5, 6, 7, 7, 9]
    assert pos[0, 1].tolist() == [0, 1, 2, 3] + [1] * 6
    assert delta.tolist() == [[0], [4 - 10]]


# ----------------------------------------------------------------------------- rot_pos
def _rot_pos_closed_form(t, h, w, m):
    out = []
    for _ in range(t):
        for bh, bw in itertools.product(range(h // m), range(w // m)):
            for ih, iw in itertools.product(range(m), range(m)):
                out.append((bh * m + ih, bw * m + iw))
    return out


@pytest.mark.parametrize("grids,m", [([(1, 4, 4)], 2), ([(2, 4, 6), (1, 2, 2)], 2),
                                     ([(1, 6, 3)], 3), ([(3, 2, 8)], 1)])
def test_rot_pos_ids_closed_form(grids, m):
    ids = oracle.rot_pos_ids_ref(torch.tensor(grids), m)
    exp = [p for (t, h, w) in grids for p in _rot_pos_closed_form(t, h, w, m)]
    assert ids.tolist() == [list(p) for p in exp]


def test_rot_pos_table_is_single_product():
    inv = wl.vision_inv_freq()
    grid = torch.tensor([[1, 32, 32], [2, 8, 12]])
    tab = oracle.rot_pos_emb_ref(inv, grid, 2)
    ids = oracle.rot_pos_ids_ref(grid, 2)
    assert tab.shape == (1024 + 192, 40) and tab.dtype == torch.float32
    exp = torch.cat([ids[:, :1].float() * inv[None], ids[:, 1:].float() * inv[None]], 1)
    assert torch.equal(tab, exp)


# ----------------------------------------------------------------------------- window_index
def _windows_brute(t, gh, gw, ws):
    """Enumerate windows by definition: (frame, window row, window col), cells row-major."""
    wins = []
    for f in range(t):
        for r0 in range(0, gh, ws):
            for c0 in range(0, gw, ws):
                wins.append([f * gh * gw + r * gw + c
                             for r in range(r0, min(r0 + ws, gh))
                             for c in range(c0, min(c0 + ws, gw))])
    return wins


@pytest.mark.parametrize("grids", [[(1, 32, 32)], [(1, 32, 32)] * 3, [(2, 10, 14), (1, 6, 22)],
                                   [(1, 2, 2)], [(3, 18, 8)]])
def test_window_index_bruteforce(grids):
    wi, cu = oracle.window_index_dedup_ref(torch.tensor(grids), 112, 2, 14, 4)
    exp_idx, exp_cu, base = [], [0], 0
    for t, h, w in grids:
        for win in _windows_brute(t, h // 2, w // 2, 4):
            exp_idx += [base + v for v in win]
            exp_cu.append(exp_cu[-1] + 4 * len(win))
        base += t * (h // 2) * (w // 2)
    assert wi.tolist() == exp_idx
    assert cu.tolist() == exp_cu
    assert sorted(wi.tolist()) == list(range(base))
    assert wi.dtype == torch.int32 and cu.dtype == torch.int32


def test_window_index_raw_list_has_duplicates_for_empty_padded_windows():
    # 16x16 merged grid is a multiple of ws = 4, so the reference pads a full extra window
    wi, cu = oracle.window_index_ref(torch.tensor([[1, 32, 32]]), 112, 2, 14, 4)
    assert len(cu) == 1 + 5 * 5 and len(set(cu)) == 1 + 16
    assert wi.dtype == torch.int64


# ----------------------------------------------------------------------------- transformers cross-check
def _hf_vision_model():
    try:
        from transformers.models.qwen2_5_vl import modeling_qwen2_5_vl as hf
    except Exception:
        pytest.skip("transformers' qwen2_5_vl module is not importable")
    return hf


def test_against_transformers_vision_helpers():
    """transformers ships the upstream functions that vl.py:473-547 were copied from; they are an
    independent implementation of the same specification (used here only, never on the GPU box path)."""
    hf = _hf_vision_model()

    class _Stub:
        spatial_merge_size = 2
        patch_size = 14
        window_size = 112
        spatial_merge_unit = 4
        rotary_pos_emb = hf.Qwen2_5_VisionRotaryEmbedding(40)

    grid = torch.tensor([[1, 32, 32], [2, 10, 14], [1, 6, 22]])
    cls = hf.Qwen2_5_VisionTransformerPretrainedModel
    try:
        wi, cu = cls.get_window_index(_Stub(), grid)
        rot = cls.rot_pos_emb(_Stub(), grid)
    except Exception as e:  # signature drift in other transformers versions
        pytest.skip(f"transformers helper not callable standalone: {e}")
    owi, ocu = oracle.window_index_ref(grid, 112, 2, 14, 4)
    assert torch.equal(wi, owi)
    # newer transformers drop the repeated entries of empty padded windows themselves
    dedup = lambda v: torch.unique_consecutive(torch.as_tensor(list(v), dtype=torch.int64)).tolist()
    assert dedup(cu) == dedup(ocu)
    if isinstance(rot, tuple):
        rot = rot[0]
    orot = oracle.rot_pos_emb_ref(_Stub.rotary_pos_emb.inv_freq, grid, 2)
    if rot.shape == orot.shape:
        assert torch.equal(rot, orot)
