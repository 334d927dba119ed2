"""CPU-side checks of the drop-in boundary: the C-ABI library loads and exports every symbol the header
declares, the ctypes table mirrors the header, and the op layer rejects bad input like the reference."""

import os
import re

import pytest
import torch

from wallx_mi355 import _lib
from wallx_mi355.fusions import ops

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "wallx_mi355.h")


def _declared():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(wx_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared()
    for must in ("wx_partition_build", "wx_permute_rows", "wx_unpermute_rows", "wx_dual_gemm",
                 "wx_dual_swiglu_ffn", "wx_mrope_apply", "wx_rope_index", "wx_rot_pos_emb", "wx_window_index"):
        assert must in names


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_lib.LIB_PATH), "libwallx_mi355.so has not been built"
    lib = _lib.load()
    for name in _declared():
        assert hasattr(lib, name), f"{name} is declared in the header but missing from the library"
    assert lib.wx_abi_version() == 1
    assert lib.wx_partition_workspace_bytes(29184) >= 29184 // 512 * 1024
    assert lib.wx_rope_index_workspace_bytes(16, 896) >= 128
    assert lib.wx_rope_index_workspace_bytes(2, 65536) >= 2 * 5 * 65536  # long rows are compacted in the workspace


def test_ctypes_table_matches_header():
    assert sorted(_lib.PROTOTYPES) == _declared()
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    for name, (_, args) in _lib.PROTOTYPES.items():
        m = re.search(name + r"\s*\((.*?)\)\s*;", text, flags=re.S)
        assert m, name
        params = m.group(1).strip()
        n = 0 if params in ("", "void") else params.count(",") + 1
        assert n == len(args), f"{name}: header has {n} parameters, ctypes table {len(args)}"


def test_argument_errors_without_a_gpu():
    # invalid arguments are rejected on the host before any launch
    lib = _lib.load()
    assert lib.wx_dual_gemm(None, None, None, None, None, None, 8, 12, 8, 0, 8, 8, 0, 1, None) == -2  # n % 8
    assert b"multiples of 8" in lib.wx_last_error_string()
    assert lib.wx_dual_gemm_add(*([None] * 8), 8, 12, 8, 0, 8, 8, 0, 1, None) == -2  # n % 8
    assert lib.wx_permute_rows(None, None, None, 4, 1, 3, _lib.WX_BF16, None) == -2  # 6-byte rows
    assert lib.wx_partition_build(None, 0, 4, 1, 300, 0, None, None, None, None, None, 0, None) == -2
    assert lib.wx_partition_build(None, 0, 4, 200, 2, 0, None, None, None, None, None, 0, None) == -2
    assert b"num_topK cannot exceed 128" in lib.wx_last_error_string()
    # a zero-width expert is refused (the MFMA kernels advance their tile loop from inside the K loop)
    assert lib.wx_dual_swiglu_ffn(*([None] * 10), 4, 64, 64, 0, None, None, None) == -2
    assert b"must be positive" in lib.wx_last_error_string()
    # host row counts that do not add up to the token count are refused
    assert lib.wx_dual_swiglu_ffn(*([None] * 10), 4, 64, 64, 64, _lib.i64x2((1, 2)), None, None) == -1
    assert b"sum to num_rows" in lib.wx_last_error_string()
    # the fused movers check their arguments the same way
    assert lib.wx_rmsnorm_permute_rows_tiled(None, None, 1e-6, None, None, None, 4, 100, None) == -2  # cols % 128
    assert lib.wx_rmsnorm_permute_rows_tiled(None, None, 1e-6, None, None, None, 4, 8192, None) == -2  # cols > 4096
    assert lib.wx_rmsnorm_permute_rows_tiled(None, None, 1e-6, None, None, None, 4, 2048, None) == -1  # null pointers
    assert lib.wx_rmsnorm_permute_rows_tiled(None, None, 1e-6, None, None, None, 0, 2048, None) == 0   # nothing to do
    assert lib.wx_unpermute_rows_add(None, None, None, None, 4, 12, None) == -2  # cols % 8
    assert lib.wx_unpermute_rows_add(None, None, None, None, 4, 16, None) == -1
    assert lib.wx_unpermute_rows_add_rmsnorm(None, None, None, None, None, 1e-6, None, 4, 8192, None) == -2  # cols > 4096
    assert lib.wx_unpermute_rows_add_rmsnorm(None, None, None, None, None, 1e-6, None, 4, 2048, None) == -1
    assert lib.wx_unpermute_rows_add_rmsnorm(None, None, None, None, None, 1e-6, None, 0, 2048, None) == 0
    assert lib.wx_rmsnorm_permute_rows(None, None, 1e-6, None, None, 4, 12, None) == -2  # cols % 8
    assert lib.wx_rmsnorm_permute_rows(None, None, 1e-6, None, None, 4, 2048, None) == -1  # null pointers
    assert lib.wx_rmsnorm_permute_rows(None, None, 1e-6, None, None, 0, 2048, None) == 0
    assert lib.wx_unpermute_rows_rmsnorm_bwd(*([None] * 3), 1e-6, *([None] * 4), 4, 8192, None, 0, None) == -2  # cols > 4096
    assert lib.wx_unpermute_rows_rmsnorm_bwd(*([None] * 3), 1e-6, *([None] * 4), 4, 2048, None, 0, None) == -1  # null pointers
    assert lib.wx_ffn_fused_workspace_bytes() >= 8
    assert lib.wx_dual_swiglu_ffn_fused(*([None] * 12), 4, 64, 64, 64, None, None, None, None) == -1  # null pointers
    assert lib.wx_dual_swiglu_ffn_fused(*([None] * 12), 0, 64, 64, 64, None, None, None, None) == 0   # nothing to do
    assert lib.wx_dual_swiglu_ffn_fused(*([None] * 12), 4, 64, 48, 64, None, None, None, None) == -2  # inter % 32
    assert lib.wx_moe_block_forward(*([None] * 13), -1, 64, 64, 64, None, None, 1e-6, 0, None, None) == -1
    assert lib.wx_moe_block_forward(*([None] * 13), 0, 64, 64, 64, None, None, 1e-6, 0, None, None) == 0   # nothing to do
    assert lib.wx_moe_block_forward(*([None] * 13), 4, 64, 64, 64, None, None, 1e-6, 0, None, None) == -1  # no sorted_row_id
    assert lib.wx_swiglu_bwd(None, None, None, None, None, None, 12, None) == -2  # count % 8
    assert lib.wx_swiglu_bwd(None, None, None, None, None, None, 16, None) == -1
    assert lib.wx_swiglu_bwd(None, None, None, None, None, None, 0, None) == 0
    assert lib.wx_swiglu_bwd_tiled(None, None, 256, None, None, None, None, 16, 96, None) == -2  # cols % 64
    assert lib.wx_swiglu_bwd_tiled(None, None, 8, None, None, None, None, 16, 64, None) == -1    # tiled_rows < rows
    assert lib.wx_swiglu_bwd_tiled(None, None, 256, None, None, None, None, 16, 64, None) == -1  # null pointers
    assert lib.wx_dual_swiglu_gate_up_keep(*([None] * 9), 4, 64, 64, 64, None, None) == -1
    assert lib.wx_dual_down_proj_residual(*([None] * 6), 4, 64, 64, 64, None, None, None) == -1  # null pointers
    assert lib.wx_dual_down_proj_residual(*([None] * 6), 0, 64, 64, 64, None, None, None) == 0   # nothing to do
    assert lib.wx_qkv_rope_proj(None, None, None, None, 48, None, 4, 64, 1, 1, 96, None) == -2
    assert b"head_dim" in lib.wx_last_error_string()
    assert lib.wx_qkv_rope_proj(None, None, None, None, 64, None, 4, 64, 1, 1, 128, None) == -1  # null pointers
    assert lib.wx_qkv_rope_proj(None, None, None, None, 96, None, 4, 64, 1, 1, 128, None) == -1
    assert b"table_width" in lib.wx_last_error_string()
    # entries per token of the packed rotary table: one per channel pair when d and d + D/2 share a position plane
    # (the PyTorch path's layout), one per channel when they do not (the CUDA kernel's layout)
    sec = _lib.i32x3((16, 24, 24))
    assert lib.wx_mrope_table_width(128, sec, _lib.WX_MROPE_HF) == 64
    assert lib.wx_mrope_table_width(128, sec, _lib.WX_MROPE_CSRC) == 128
    assert lib.wx_mrope_table_width(128, _lib.i32x3((64, 0, 0)), _lib.WX_MROPE_CSRC) == 64  # one plane: the maps agree
    assert lib.wx_mrope_table_width(128, _lib.i32x3((16, 24, 25)), _lib.WX_MROPE_HF) == -1
    assert lib.wx_mrope_table(None, None, 1, 4, 128, sec, _lib.WX_MROPE_CSRC, None, None) == -1  # null pointers
    assert lib.wx_partition_build_noalloc(None, 0, 4, 200, 2, 0, None, None, None, None, None) == -2
    # M-RoPE from positions: shapes the row kernel cannot take are refused, not routed elsewhere
    st = _lib.i64x3((128 * 4, 128, 128 * 4))
    assert lib.wx_mrope_apply_positions(None, None, None, None, None, None, 1, 4, 2, 1, 128, st, st, st, st,
                                        _lib.i32x3((10, 27, 27)), 0, _lib.WX_BF16, 0, None) == -1  # null pointers
    q = torch.zeros(8)
    p_ = q.data_ptr()  # never dereferenced: the call fails on the host
    assert lib.wx_mrope_apply_positions(p_, p_, p_, p_, p_, p_, 1, 4, 2, 1, 128, st, st, st, st,
                                        _lib.i32x3((10, 27, 27)), 0, _lib.WX_BF16, 0, None) == -2
    assert b"chunk boundaries" in lib.wx_last_error_string()


def test_op_layer_validation_matches_reference_behaviour():
    x = torch.randn(4, 8)
    with pytest.raises(RuntimeError, match="on the device: CPU"):
        ops.permute(x, torch.zeros(4, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="on the device: CPU"):
        ops.unpermute(x, torch.zeros(4, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="on the device: CPU"):
        ops.multimodal_rope(x, x, x, x, [1, 1, 2])
    # empty input short-circuits (ops.py:194-195, 294-296)
    e = torch.empty(0, 8)
    out, rmap = ops.permute(e, torch.zeros(0, dtype=torch.int32))
    assert out.shape == e.shape and rmap is None
    assert ops.unpermute(e, torch.zeros(0, dtype=torch.int32)).shape == e.shape
    with pytest.raises(TypeError):
        ops.get_rope_index([1, 2], 2, 1, 2, 3, 2)
    with pytest.raises(ValueError, match="2D"):
        ops.get_rope_index(torch.zeros(4, dtype=torch.long), 2, 1, 2, 3, 2)
    with pytest.raises(ValueError, match="CUDA"):
        ops.get_rope_index(torch.zeros(1, 4, dtype=torch.long), 2, 1, 2, 3, 2)
    with pytest.raises(TypeError):
        ops.rot_pos_emb([1.0], torch.zeros(1, 3, dtype=torch.long), 2)
    with pytest.raises(ValueError, match="1-dimensional"):
        ops.rot_pos_emb(torch.zeros(2, 2), torch.zeros(1, 3, dtype=torch.long), 2)
    with pytest.raises(ValueError, match=r"\[num_grids, 3\]"):
        ops.rot_pos_emb(torch.zeros(2), torch.zeros(1, 2, dtype=torch.long), 2)
    with pytest.raises(AssertionError):
        ops.get_window_index(torch.zeros(3, dtype=torch.int32), 112, 2, 14, 4)
    with pytest.raises(AssertionError, match="2D"):
        ops.asym_dual_gmm(torch.zeros(2), torch.zeros(2, 2), torch.zeros(2, 2), torch.zeros(2, 2))
    with pytest.raises(AssertionError, match="dimension mismatch"):
        ops.asym_dual_gmm(torch.zeros(2, 3), torch.zeros(2, 2), torch.zeros(2, 2), torch.zeros(2, 2))


def test_wallx_csrc_shim_exposes_the_nine_native_names():
    import wallx_csrc

    for name in ("asym_dual_gmm", "permute", "unpermute", "unpermute_bwd", "rope", "rope_bwd", "rope_index",
                 "rot_pos_emb", "get_window_index"):
        assert callable(getattr(wallx_csrc, name))
