"""CPU oracle for the wall-x per-layer MoE hot path.

THIS PACKAGE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, in plain
torch/numpy on the CPU, the algorithms of the reference's PyTorch path so that
the HIP kernels can be checked against them.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it; nothing under the product package does, and the product fails
loudly when its HIP library is missing rather than falling back to this code.

Every function cites the reference file:line it follows.  Abbreviations:

  act.py = wall_x/model/qwen2_5_based/modeling_qwen2_5_vl_act.py
  vl.py  = wall_x/model/qwen2_5_based/modeling_qwen2_5_vl.py
  ops.py = wall_x/fusions/ops.py

How each function is pinned (tests/test_oracle_*.py):

  permute_ref / unpermute_ref      brute-force stable partition on tiny inputs,
                                   round-trip identity, permutation invariants
  dual_gemm_ref / swiglu_ffn_ref   float64 numpy contraction on small shapes,
                                   linearity, zero-row groups; the gelu / relu
                                   gated forms and a three-expert block against a
                                   float64 scalar-loop evaluation with math.erf
  mrope_apply_ref                  textbook rotate-half RoPE when t == h == w,
                                   identity at position 0, per-pair norm
                                   preservation, transformers' same-lineage
                                   function where it is importable
  rotary_cos_sin_ref               closed form cos(pos * inv_freq)
  rope_index_ref                   the known-answer vector in the reference
                                   docstring (vl.py:1744-1760), closed form of
                                   the camera/text/action layout, text-only
                                   cumsum branch
  rot_pos_ids_ref / rot_pos_emb_ref  closed form (h, w) of the merge-block order,
                                   brute force over small grids
  window_index_ref                 permutation / window-size invariants, brute
                                   force enumeration of windows on small grids
  swiglu_bwd_ref                   central differences of silu(g) * u in float64,
                                   the closed form of silu' at 0 and far from 0
  rms_norm_ref                     torch.nn.functional.rms_norm in fp32, the
                                   closed form for constant rows, transformers'
                                   Qwen2RMSNorm where it is importable

  unpermute_ref with topK > 1      the fp32 weighted sum x * sum_k p; in bf16 the
                                   exactly representable cases and a bound of one
                                   rounding per operation
  unpermute_bwd_ref                torch autograd of the scalar-loop expression
                                   out[t] = sum_k p[t,k] y[map[k*T+t]] on tiny
                                   inputs (with dropped rows), the adjoint identity
  mrope_apply_ref(layout="csrc")   per-channel closed form with distinct t / h / w
                                   positions and the plane thresholds written out
                                   from csrc/rope.cu:104-117

  One aspect no CPU fact can fix: WHERE the reference's CUDA kernels round to
  bf16 inside a topK > 1 combine (csrc/permute.cu:69-154 rounds every product and
  every partial sum).  The oracle follows that source; the tests above bound the
  effect (one rounding per operation) and wall-x itself only ever runs topK == 1,
  where the ops are bit copies.
"""

from .permute import (  # noqa: F401
    permute_ref,
    unpermute_ref,
    unpermute_bwd_ref,
    expert_offsets_ref,
)
from .ffn import activation_ref, dual_gemm_ref, swiglu_ffn_ref, swiglu_bwd_ref, sparse_moe_block_ref  # noqa: F401
from .mrope import (  # noqa: F401
    rotate_half_ref,
    mrope_axis_map,
    mrope_apply_ref,
    mrope_apply_bwd_ref,
    rotary_cos_sin_ref,
)
from .rope_index import rope_index_ref  # noqa: F401
from .rot_pos import rot_pos_ids_ref, rot_pos_emb_ref  # noqa: F401
from .window_index import window_index_ref, window_index_dedup_ref  # noqa: F401
from .norm import rms_norm_ref  # noqa: F401
