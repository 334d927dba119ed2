"""Oracle: 3D M-RoPE position ids (test infrastructure only).

Restates Qwen2_5_VLMoEForAction.get_rope_index (act.py:929-1149; an identical
copy lives at vl.py:1721-1940) with numpy on the host.  Integer output; the
HIP kernel must match it bit for bit.
"""

import numpy as np
import torch


class RopeIndexInputError(ValueError):
    """The reference would raise (ValueError from list.index, IndexError, or a
    shape mismatch on assignment) for this input."""


def _walk_row(tokens, image_id, video_id, vstart_id, merge, tps,
              image_grid, video_grid, sec_per_grid, img_i, vid_i):
    """Positions [3, L] for one unpadded row; returns (pos, img_i, vid_i)."""
    L = len(tokens)
    toks = np.asarray(tokens, dtype=np.int64)
    # act.py:995-1000: a vision item is a <vision_start> followed by an image/video token
    starts = np.nonzero(toks == vstart_id)[0]
    if len(starts) and starts[-1] + 1 >= L:
        raise RopeIndexInputError("vision_start is the last token")
    follow = toks[starts + 1] if len(starts) else np.zeros(0, np.int64)
    n_img = int((follow == image_id).sum())
    n_vid = int((follow == video_id).sum())
    tok_list = toks.tolist()
    has_img = image_id in tok_list
    has_vid = video_id in tok_list

    chunks = []
    st = 0
    last_max = None  # max of the most recent chunk (always a vision chunk when read)
    rem_img, rem_vid = n_img, n_vid
    for _ in range(n_img + n_vid):
        # act.py:1010-1018
        if has_img and rem_img > 0:
            try:
                ed_img = tok_list.index(image_id, st)
            except ValueError as e:
                raise RopeIndexInputError(str(e))
        else:
            ed_img = L + 1
        if has_vid and rem_vid > 0:
            try:
                ed_vid = tok_list.index(video_id, st)
            except ValueError as e:
                raise RopeIndexInputError(str(e))
        else:
            ed_vid = L + 1
        if ed_img < ed_vid:  # act.py:1021-1031
            t, h, w = (int(v) for v in image_grid[img_i])
            spg = None  # images: second_per_grid_t = 0 (integer zero)
            img_i += 1
            rem_img -= 1
            ed = ed_img
        else:  # act.py:1032-1045
            t, h, w = (int(v) for v in video_grid[vid_i])
            spg = np.float32(sec_per_grid[vid_i]) if sec_per_grid is not None else np.float32(1.0)
            vid_i += 1
            rem_vid -= 1
            ed = ed_vid
        gt, gh, gw = t, h // merge, w // merge  # act.py:1048-1052
        text_len = ed - st
        st_idx = 0 if last_max is None else last_max + 1  # act.py:1056-1060
        text = np.arange(text_len, dtype=np.int64) + st_idx
        chunks.append(np.stack([text, text, text]))
        # act.py:1066-1076: t index = trunc(fp32(t) * second_per_grid * tokens_per_second)
        tt = np.repeat(np.arange(gt, dtype=np.int64), gh * gw)
        if spg is None:
            t_idx = np.zeros_like(tt)
        else:
            f = tt.astype(np.float32) * spg          # int64 tensor * 0-dim fp32 tensor -> fp32
            f = f * np.float32(tps)                   # fp32 tensor * python scalar -> fp32
            t_idx = np.trunc(f).astype(np.int64)      # .long()
        h_idx = np.tile(np.repeat(np.arange(gh, dtype=np.int64), gw), gt)
        w_idx = np.tile(np.arange(gw, dtype=np.int64), gt * gh)
        vis = np.stack([t_idx, h_idx, w_idx]) + text_len + st_idx  # act.py:1093-1095
        if vis.shape[1] == 0:
            raise RopeIndexInputError("empty vision grid")  # .max() of an empty tensor
        chunks.append(vis)
        last_max = int(vis.max())
        st = ed + gt * gh * gw  # act.py:1096
    if st < L:  # act.py:1099-1108
        st_idx = 0 if last_max is None else last_max + 1
        text = np.arange(L - st, dtype=np.int64) + st_idx
        chunks.append(np.stack([text, text, text]))
    if not chunks:
        raise RopeIndexInputError("row with no unmasked tokens")  # torch.cat([]) raises
    pos = np.concatenate(chunks, axis=1)
    if pos.shape[1] != L:
        raise RopeIndexInputError(f"positions {pos.shape[1]} != tokens {L}")  # act.py:1112
    return pos, img_i, vid_i


def rope_index_ref(input_ids, spatial_merge_size, image_token_id, video_token_id,
                   vision_start_token_id, tokens_per_second, image_grid_thw=None,
                   video_grid_thw=None, second_per_grid_ts=None, attention_mask=None):
    """Returns (position_ids [3,B,S] int64, mrope_position_deltas [B,1] int64)."""
    ids = input_ids.cpu().numpy().astype(np.int64)
    B, S = ids.shape
    if image_grid_thw is None and video_grid_thw is None:
        # act.py:1123-1149 text-only branch
        if attention_mask is not None:
            m = attention_mask.cpu().numpy().astype(np.int64)
            p = np.cumsum(m, axis=-1) - 1
            p[m == 0] = 1
            pos = np.broadcast_to(p[None], (3, B, S)).copy()
            delta = p.max(axis=-1, keepdims=True) + 1 - S
        else:
            pos = np.broadcast_to(np.arange(S, dtype=np.int64)[None, None], (3, B, S)).copy()
            delta = np.zeros((B, 1), dtype=np.int64)
        return torch.from_numpy(pos), torch.from_numpy(delta.astype(np.int64))

    mask = (np.ones_like(ids) if attention_mask is None
            else attention_mask.cpu().numpy().astype(np.int64))
    ig = None if image_grid_thw is None else image_grid_thw.cpu().numpy().astype(np.int64)
    vg = None if video_grid_thw is None else video_grid_thw.cpu().numpy().astype(np.int64)
    spg = None if second_per_grid_ts is None else second_per_grid_ts.cpu().numpy().astype(np.float32)
    pos = np.ones((3, B, S), dtype=np.int64)  # act.py:978-984
    deltas = np.zeros((B, 1), dtype=np.int64)
    img_i = vid_i = 0  # act.py:986: the grid cursors run across the whole batch
    for b in range(B):
        keep = mask[b] == 1  # act.py:991
        row, img_i, vid_i = _walk_row(ids[b][keep].tolist(), image_token_id, video_token_id,
                                      vision_start_token_id, spatial_merge_size,
                                      tokens_per_second, ig, vg, spg, img_i, vid_i)
        pos[:, b, keep] = row  # act.py:1112
        deltas[b, 0] = row.max() + 1 - S  # act.py:1115-1117
    return torch.from_numpy(pos), torch.from_numpy(deltas)
