"""Oracle: vision-tower window attention index (test infrastructure only).

Restates Qwen2_5_VisionTransformerPretrainedModel.get_window_index
(vl.py:502-547) with numpy.
"""

import numpy as np
import torch


def window_index_ref(grid_thw, window_size: int, spatial_merge_size: int, patch_size: int,
                     spatial_merge_unit: int):
    """Returns (window_index int64 [N], cu_window_seqlens python list).

    vl.py:506-508: ws = window_size // merge // patch.  Each merged frame
    [t, h/m, w/m] is padded with -100 on the bottom/right by ``ws - x % ws``
    (a full extra window when x is already a multiple, vl.py:518-519), cut into
    ws x ws windows ordered (t, win_row, win_col), and the padding dropped.  The
    cumulative list therefore repeats an entry for every empty window.
    """
    ws = window_size // spatial_merge_size // patch_size
    index_parts = []
    cu = [0]
    base = 0
    for t, h, w in np.asarray(grid_thw.cpu()).astype(np.int64).tolist():
        gh, gw = h // spatial_merge_size, w // spatial_merge_size
        idx = np.arange(t * gh * gw, dtype=np.int64).reshape(t, gh, gw)
        pad_h = ws - gh % ws
        pad_w = ws - gw % ws
        nh, nw = (gh + pad_h) // ws, (gw + pad_w) // ws
        padded = np.full((t, gh + pad_h, gw + pad_w), -100, dtype=np.int64)
        padded[:, :gh, :gw] = idx
        win = padded.reshape(t, nh, ws, nw, ws).transpose(0, 1, 3, 2, 4).reshape(t, nh * nw, ws, ws)
        seqlens = (win != -100).sum(axis=(2, 3)).reshape(-1)
        flat = win.reshape(-1)
        index_parts.append(flat[flat != -100] + base)
        cu.extend((np.cumsum(seqlens) * spatial_merge_unit + cu[-1]).tolist())  # vl.py:540-543
        base += t * gh * gw
    if index_parts:
        window_index = torch.from_numpy(np.concatenate(index_parts))
    else:
        window_index = torch.zeros(0, dtype=torch.int64)
    return window_index, cu


def window_index_dedup_ref(grid_thw, window_size: int, spatial_merge_size: int, patch_size: int,
                           spatial_merge_unit: int):
    """(window_index int32 [N], cu_window_seqlens int32 [W+1]) as the fused op returns them
    (ops.py:685-742, csrc/window_index.cu:208-286): int32, and one cumulative
    entry per non-empty window, i.e. unique_consecutive of the list above.
    """
    wi, cu = window_index_ref(grid_thw, window_size, spatial_merge_size, patch_size,
                              spatial_merge_unit)
    cu_t = torch.unique_consecutive(torch.tensor(cu, dtype=torch.int64))
    return wi.to(torch.int32), cu_t.to(torch.int32)
