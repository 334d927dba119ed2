"""Mirror of wall_x/fusions/backend.py: thin forwarding layer between ops.py and the native entry points.

Function names, argument order and defaults follow the reference (backend.py:71-433) so code written
against ``wall_x.fusions.backend`` keeps working; the native module is ``wallx_mi355.native``.
"""

from typing import Optional, Tuple

import torch

from .. import native


def asym_dual_gmm_separated(input_expert0, input_expert1, weight_expert0, weight_expert1,
                            output_expert0: Optional[torch.Tensor] = None,
                            output_expert1: Optional[torch.Tensor] = None,
                            trans_a: bool = False, trans_b: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """backend.py:71-135.  Missing outputs are allocated as [m_e, n_e] in the input dtype."""

    def out_shape(a, w):
        m = a.size(1) if trans_a else a.size(0)
        n = w.size(0) if trans_b else w.size(1)
        return m, n

    if output_expert0 is None:
        output_expert0 = torch.empty(out_shape(input_expert0, weight_expert0), device=input_expert0.device,
                                     dtype=input_expert0.dtype)
    if output_expert1 is None:
        output_expert1 = torch.empty(out_shape(input_expert1, weight_expert1), device=input_expert1.device,
                                     dtype=input_expert1.dtype)
    native.asym_dual_gmm(input_expert0, input_expert1, weight_expert0, weight_expert1, output_expert0,
                         output_expert1, trans_a, trans_b)
    return output_expert0, output_expert1


def permute(input, indices, num_out_tokens, workspace, max_expanded_token_num):
    """backend.py:138-167 -> (permuted, row_id_map, workspace)."""
    return native.permute(input, indices, num_out_tokens, workspace, max_expanded_token_num)


def unpermute(input, row_id_map, prob, max_tokens, num_topK):
    """backend.py:170-197."""
    return native.unpermute(input, row_id_map, prob, max_tokens, num_topK)


def unpermute_bwd(input_bwd, input_fwd, row_id_map, prob):
    """backend.py:200-230: prob None means uniform weights of one expert per token."""
    if prob is None:
        prob = torch.ones([input_bwd.size(0), 1], dtype=torch.float32, device=input_bwd.device)
    return native.unpermute_bwd(input_bwd, input_fwd, row_id_map, prob)


def rope(q, k, cos, sin, q_out, k_out, mrope_section_doubled, layout: str = "csrc") -> None:
    """backend.py:233-262.  layout: "csrc" = the channel map of the reference's kernel, "hf" = its PyTorch path."""
    return native.rope(q, k, cos, sin, q_out, k_out, mrope_section_doubled, layout)


def rope_bwd(grad_q_out, grad_k_out, q, k, cos, sin, grad_q, grad_k, mrope_section_doubled,
             layout: str = "csrc") -> None:
    """backend.py:265-299."""
    return native.rope_bwd(grad_q_out, grad_k_out, q, k, cos, sin, grad_q, grad_k, mrope_section_doubled, layout)


def rope_from_positions(q, k, position_ids, inv_freq, q_out, k_out, mrope_section_doubled, backward=False,
                        layout: str = "hf") -> None:
    """No counterpart in backend.py: the rope op with the cos/sin builder (vl.py:679-712) folded in."""
    return native.rope_from_positions(q, k, position_ids, inv_freq, q_out, k_out, mrope_section_doubled, backward,
                                      layout)


def rope_from_table(q, k, table, q_out, k_out, mrope_section_doubled, backward=False, layout: str = "hf") -> None:
    """No counterpart in backend.py: the rope op reading the packed cos/sin table of mrope_table."""
    return native.rope_from_table(q, k, table, q_out, k_out, mrope_section_doubled, backward, layout)


def mrope_table(position_ids, inv_freq, mrope_section, layout: str = "hf"):
    """No counterpart in backend.py: the packed cos/sin table the projection below reads (vl.py:679-712)."""
    return native.mrope_table(position_ids, inv_freq, mrope_section, layout)


def qkv_rope_proj(x, weight, bias, table, n_q_heads, n_kv_heads, head_dim=128, out=None):
    """No counterpart in backend.py: q / k / v projections with the rotary embedding in the epilogue (vl.py:955-964)."""
    return native.qkv_rope_proj(x, weight, bias, table, n_q_heads, n_kv_heads, head_dim, out)


def get_rope_index(input_ids, image_grid_thw, video_grid_thw, second_per_grid_ts, attention_mask,
                   spatial_merge_size, image_token_id, video_token_id, vision_start_token_id, tokens_per_second):
    """backend.py:302-352 (forwards to the native op named rope_index)."""
    return native.rope_index(input_ids, image_grid_thw, video_grid_thw, second_per_grid_ts, attention_mask,
                             spatial_merge_size, image_token_id, video_token_id, vision_start_token_id,
                             tokens_per_second)


def rot_pos_emb(inv_freq, grid_thw, spatial_merge_size, grid_thw_host=None):
    """backend.py:355-387."""
    return native.rot_pos_emb(inv_freq, grid_thw, spatial_merge_size, grid_thw_host=grid_thw_host)


def get_window_index(grid_thw, spatial_merge_size, vit_merger_window_size, patch_size, spatial_merge_unit,
                     grid_thw_host=None):
    """backend.py:390-433."""
    return native.get_window_index(grid_thw, spatial_merge_size, vit_merger_window_size, patch_size,
                                   spatial_merge_unit, grid_thw_host=grid_thw_host)
