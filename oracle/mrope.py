"""Oracle: 3D multimodal RoPE (test infrastructure only).

Follows vl.py:215-219 (rotate_half), vl.py:731-773
(apply_multimodal_rotary_pos_emb) and vl.py:679-712 (cos/sin builder).  The
reference's CUDA kernel (csrc/rope.cu:104-117) assigns channels to the t/h/w
axes differently; that layout is available as layout="csrc".
"""

import torch


def rotate_half_ref(x):
    # vl.py:215-219: (x1, x2) -> (-x2, x1) over the two halves of the last dim
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def mrope_axis_map(mrope_section, head_dim: int, layout: str = "hf"):
    """axis[d] in {0,1,2} (t, h, w) for every channel d.

    layout "hf":  vl.py:763-769 -- the section list is doubled by *list
      repetition* ([16,24,24] -> [16,24,24,16,24,24]) and chunk i takes axis i % 3.
    layout "csrc": csrc/rope.cu:104-117 with ops.py:451 -- the sections are
      doubled *elementwise* ([32,48,48]) and laid out contiguously t, h, w.
    """
    if layout == "hf":
        chunks = list(mrope_section) * 2
        axes = []
        for i, n in enumerate(chunks):
            axes += [i % 3] * n
    elif layout == "csrc":
        s0, s1, _ = [2 * v for v in mrope_section]
        axes = [0 if d < s0 else (1 if d < s0 + s1 else 2) for d in range(head_dim)]
    else:
        raise ValueError(layout)
    if len(axes) != head_dim:
        raise ValueError(f"mrope_section {mrope_section} does not cover head_dim {head_dim}")
    return torch.tensor(axes, dtype=torch.long)


def _select(table, axis_map):
    # table [3, B, S, D] -> [B, S, D] with channel d taken from plane axis_map[d]
    D = table.shape[-1]
    return table[axis_map, :, :, torch.arange(D)].permute(1, 2, 0)


def mrope_apply_ref(q, k, cos, sin, mrope_section, layout: str = "hf", eager_rounding: bool = True):
    """q' = q*cos_sel + rotate_half(q)*sin_sel (same for k); vl.py:771-772.

    q [B, Hq, S, D], k [B, Hkv, S, D], cos/sin [3, B, S, D].
    eager_rounding=True evaluates op by op in q.dtype as eager PyTorch does
    (each product and the sum are rounded to the storage dtype);
    False computes in fp32 and rounds once.
    """
    D = q.shape[-1]
    amap = mrope_axis_map(mrope_section, D, layout)
    c = _select(cos, amap).unsqueeze(1)  # [B, 1, S, D]  (unsqueeze_dim = 1)
    s = _select(sin, amap).unsqueeze(1)
    if eager_rounding:
        return (q * c) + (rotate_half_ref(q) * s), (k * c) + (rotate_half_ref(k) * s)
    c32, s32 = c.float(), s.float()

    def one(x):
        x32 = x.float()
        return (x32 * c32 + rotate_half_ref(x32) * s32).to(x.dtype)

    return one(q), one(k)


def mrope_apply_bwd_ref(gq, gk, cos, sin, mrope_section, layout: str = "hf"):
    """Adjoint of mrope_apply_ref w.r.t. q and k (fp32 math, one rounding):
    g_in = g*cos_sel + rotate_half^T(g*sin_sel), rotate_half^T(y) = (y2, -y1).
    csrc/rope.cu:274-314 computes the same expression channel by channel.
    """
    D = gq.shape[-1]
    amap = mrope_axis_map(mrope_section, D, layout)
    c = _select(cos, amap).unsqueeze(1).float()
    s = _select(sin, amap).unsqueeze(1).float()
    half = D // 2

    def one(g):
        g32 = g.float()
        ys = g32 * s
        rt = torch.cat((ys[..., half:], -ys[..., :half]), dim=-1)
        return (g32 * c + rt).to(g.dtype)

    return one(gq), one(gk)


def rotary_cos_sin_ref(position_ids, inv_freq, dtype, attention_scaling: float = 1.0):
    """cos/sin [3, B, S, D] from position_ids [3, B, S] (vl.py:679-712).

    freqs = pos (fp32) * inv_freq (fp32) via an fp32 matmul with inner size 1,
    emb = cat(freqs, freqs), cos/sin in fp32, scaled, cast to the activation dtype.
    """
    pos = position_ids.to(torch.float32)
    freqs = pos[..., None] * inv_freq.to(torch.float32)[None, None, None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return (emb.cos() * attention_scaling).to(dtype), (emb.sin() * attention_scaling).to(dtype)
