"""Seeded synthetic inputs at the shapes the hot path is measured on.

Everything is generated on the CPU from an explicit torch.Generator so that the
GPU path and a CPU checker see identical bits; callers move tensors to the
device themselves.  Token layout follows the reference's prompt builder
(wall_x/data/utils.py:453-503: per camera ``<vision_start><image_pad>*n
<vision_end>``, text, then ``<|action|>`` * chunk) and its gating rule
(wall_x/data/load_lerobot_dataset.py:406-409: moe_token_types = ids == action id).
"""

from dataclasses import dataclass

import torch

# Qwen2.5-VL special-token ids (the reference reads them from the checkpoint
# config, act.py:965-967, and ships no values; any distinct ints work).
IMAGE_TOKEN_ID = 151655
VIDEO_TOKEN_ID = 151656
VISION_START_TOKEN_ID = 151652
VISION_END_TOKEN_ID = 151653
ACTION_TOKEN_ID = 151666
TEXT_TOKEN_ID = 1000

HIDDEN = 2048
INTER_VL = 11008
INTER_ACT = 1024
HEAD_DIM = 128
N_Q_HEADS = 16
N_KV_HEADS = 2
MROPE_SECTION = (16, 24, 24)
ROPE_THETA = 1.0e6


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def randn(shape, std: float, dtype, gen) -> torch.Tensor:
    return (torch.randn(shape, generator=gen, dtype=torch.float32) * std).to(dtype)


@dataclass
class ExpertWeights:
    gate: torch.Tensor  # [I, H]  nn.Linear layout (act.py:74)
    up: torch.Tensor    # [I, H]
    down: torch.Tensor  # [H, I]

    def to(self, device):
        return ExpertWeights(self.gate.to(device), self.up.to(device), self.down.to(device))

    def as_tuple(self):
        return (self.gate, self.up, self.down)


def expert_weights(hidden, inter, dtype, gen, std=0.02) -> ExpertWeights:
    return ExpertWeights(randn((inter, hidden), std, dtype, gen),
                         randn((inter, hidden), std, dtype, gen),
                         randn((hidden, inter), std, dtype, gen))


def moe_layer_inputs(n_seq, seq_len, n_action, dtype, seed=0, mask="random",
                     hidden=HIDDEN, inter=(INTER_VL, INTER_ACT), w_std=0.02):
    """hidden [n_seq, seq_len, H], token types [n_seq, seq_len] bool, two experts' weights.

    mask="random": per row, a seeded random permutation places exactly n_action
    action tokens; mask="tail": the last n_action tokens of the row are action tokens.
    """
    g = _gen(seed)
    x = randn((n_seq, seq_len, hidden), 1.0, dtype, g)
    types = torch.zeros(n_seq, seq_len, dtype=torch.bool)
    for b in range(n_seq):
        if mask == "random":
            types[b, torch.randperm(seq_len, generator=g)[:n_action]] = True
        else:
            types[b, seq_len - n_action:] = True
    weights = [expert_weights(hidden, inter[0], dtype, g, w_std),
               expert_weights(hidden, inter[1], dtype, g, w_std)]
    return x, types, weights


def config1(seed=0):
    """512 fp32 tokens, the first 448 to the VL expert and the last 64 to the action expert."""
    return moe_layer_inputs(1, 512, 64, torch.float32, seed, mask="tail")


def config3(seed=0, n_seq=32):
    """bf16 serving batch: n_seq x 912 tokens, 880 VL + 32 action per sequence."""
    return moe_layer_inputs(n_seq, 912, 32, torch.bfloat16, seed, mask="random")


def vla_row_tokens(n_images=3, image_tokens=256, lead_text=10, tail_text=80, n_action=32):
    row = [TEXT_TOKEN_ID] * lead_text
    for _ in range(n_images):
        row += [VISION_START_TOKEN_ID] + [IMAGE_TOKEN_ID] * image_tokens + [VISION_END_TOKEN_ID]
    row += [TEXT_TOKEN_ID] * tail_text + [ACTION_TOKEN_ID] * n_action
    return row


def config2_tokens(batch=16, tail_text=80):
    """input_ids [batch, S] int64 and image_grid_thw [3*batch, 3] int64.

    Three 448x448 camera images per row, patch 14 -> grid (1, 32, 32), 2x2 merge
    -> 256 image tokens each; S = 896 with tail_text = 80 (96 text-class tokens
    including the six vision delimiters) and S = 912 with tail_text = 96.
    """
    row = vla_row_tokens(tail_text=tail_text)
    ids = torch.tensor([row] * batch, dtype=torch.int64)
    grid = torch.tensor([[1, 32, 32]] * (3 * batch), dtype=torch.int64)
    return ids, grid


def vision_inv_freq(head_dim=80, theta=10000.0):
    """Qwen2.5-VL ViT: hidden 1280 / 16 heads = 80, rotary dim = head_dim // 2 (vl.py:457-458,111)."""
    dim = head_dim // 2
    return 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float) / dim))


def text_inv_freq(head_dim=HEAD_DIM, theta=ROPE_THETA):
    return 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float) / head_dim))


def qk_inputs(batch, seq_len, dtype=torch.bfloat16, seed=0):
    """Token-major q [B, S, Hq, D] and k [B, S, Hkv, D] as the attention projections produce them."""
    g = _gen(seed)
    q = randn((batch, seq_len, N_Q_HEADS, HEAD_DIM), 1.0, dtype, g)
    k = randn((batch, seq_len, N_KV_HEADS, HEAD_DIM), 1.0, dtype, g)
    return q, k
