"""wallx_mi355: the wall-x per-layer MoE hot path on MI355X (gfx950).

    wallx_mi355.fusions.ops      the seven ops of wall_x.fusions.ops, same signatures
    wallx_mi355.native           the nine native entry points of the reference's wallx_csrc module
    wallx_mi355.moe              SparseMoeBlock-compatible block on the fused dual-expert FFN
    wallx_mi355.workloads        seeded synthetic inputs at the measured shapes

All computation happens in libwallx_mi355.so (hand-written HIP, C ABI in include/wallx_mi355.h).
"""

from . import _lib  # noqa: F401

__version__ = "0.1.0"
