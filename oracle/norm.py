"""RMSNorm as the decoder layer applies it (act.py:190-193, 256-258: `post_attention_layernorm` is a
Qwen2RMSNorm; the class comes from transformers, act.py:23-25).  Test infrastructure only.

Restated from the published module: the input is upcast to fp32, variance = mean(x^2) over the last axis,
x * rsqrt(variance + eps) is cast back to the input dtype and multiplied by the weight (in the weight's dtype).
Pinned in tests/test_oracle_float.py against torch.nn.functional.rms_norm in fp32 (a library routine), the closed
form for constant rows, and transformers' own Qwen2RMSNorm where that module imports.
"""

import torch


def rms_norm_ref(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    h = x.to(torch.float32)
    variance = h.pow(2).mean(-1, keepdim=True)
    h = h * torch.rsqrt(variance + eps)
    return weight * h.to(x.dtype)
