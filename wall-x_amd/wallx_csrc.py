"""Drop-in for the reference's compiled extension module ``wallx_csrc`` (csrc/ops.cu:11-21).

The reference's ``wall_x/fusions/backend.py`` does ``import wallx_csrc as backend`` (backend.py:13); with this
directory on ``sys.path`` that import resolves here and the reference's own ops.py / backend.py / model code
run unchanged on the MI355X kernels.
"""

from wallx_mi355.native import (  # noqa: F401
    asym_dual_gmm,
    get_window_index,
    permute,
    rope,
    rope_bwd,
    rope_index,
    rot_pos_emb,
    unpermute,
    unpermute_bwd,
)

__all__ = ["asym_dual_gmm", "permute", "unpermute", "unpermute_bwd", "rope", "rope_bwd", "rope_index",
           "rot_pos_emb", "get_window_index"]
