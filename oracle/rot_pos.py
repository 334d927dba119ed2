"""Oracle: vision-tower rotary position ids and table (test infrastructure only).

Restates Qwen2_5_VisionTransformerPretrainedModel.rot_pos_emb (vl.py:473-500)
and Qwen2_5_VisionRotaryEmbedding (vl.py:108-119).
"""

import numpy as np
import torch


def rot_pos_ids_ref(grid_thw, spatial_merge_size: int) -> torch.Tensor:
    """[sum t*h*w, 2] int64 (h_pos, w_pos) per patch, patches in merge-block order.

    vl.py:475-495: the (h, w) coordinate planes are cut into m x m blocks
    (reshape to [h/m, m, w/m, m], swap the middle axes) so the m*m patches that
    the merger fuses are adjacent; the frame is repeated t times.
    """
    m = spatial_merge_size
    out = []
    for t, h, w in np.asarray(grid_thw.cpu()).astype(np.int64).tolist():
        hh = np.broadcast_to(np.arange(h)[:, None], (h, w))
        ww = np.broadcast_to(np.arange(w)[None, :], (h, w))

        def blocked(a):
            return a.reshape(h // m, m, w // m, m).transpose(0, 2, 1, 3).reshape(-1)

        frame = np.stack([blocked(hh), blocked(ww)], axis=-1)
        out.append(np.tile(frame, (t, 1)))
    if not out:
        return torch.zeros(0, 2, dtype=torch.int64)
    return torch.from_numpy(np.concatenate(out, 0).astype(np.int64))


def rot_pos_emb_ref(inv_freq: torch.Tensor, grid_thw, spatial_merge_size: int) -> torch.Tensor:
    """[N, 2F] fp32: row n = [h_pos*inv_freq, w_pos*inv_freq] (vl.py:496-499).

    The reference builds outer(arange(max_grid), inv_freq) in fp32 and gathers
    rows with the ids; each entry is a single fp32 product.
    """
    ids = rot_pos_ids_ref(grid_thw, spatial_merge_size)
    g = np.asarray(grid_thw.cpu()).astype(np.int64)
    max_grid = int(g[:, 1:].max()) if len(g) else 0
    seq = torch.arange(max_grid, dtype=torch.float32)
    table = torch.outer(seq, inv_freq.to(torch.float32).cpu())  # vl.py:114-119
    return table[ids].flatten(1)
