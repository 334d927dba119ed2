"""ctypes binding of libwallx_mi355.so (the C ABI declared in include/wallx_mi355.h).

The library is built in-tree by ``wall-x_amd/csrc/build.py``; there is no fallback path: if it is
missing, loading raises.
"""

import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
# WALLX_MI355_LIB points at an alternative build of the same library (e.g. one compiled with other tuning flags)
LIB_PATH = os.environ.get("WALLX_MI355_LIB") or os.path.join(_HERE, "libwallx_mi355.so")

WX_F32, WX_F16, WX_BF16 = 0, 1, 2
WX_I32, WX_I64, WX_U8 = 0, 1, 2
WX_MROPE_HF, WX_MROPE_CSRC = 0, 1
WX_GEMM_PATH_MFMA, WX_GEMM_PATH_ZERO_FILL, WX_GEMM_PATH_FMA, WX_GEMM_PATH_ADD_COPY = 1, 2, 4, 8

_c = ctypes
_vp, _i64, _i32, _sz, _f32 = _c.c_void_p, _c.c_int64, _c.c_int, _c.c_size_t, _c.c_float

# name -> (restype, argtypes); mirrors include/wallx_mi355.h one to one
PROTOTYPES = {
    "wx_last_error_string": (_c.c_char_p, []),
    "wx_last_gemm_path": (_i32, []),
    "wx_abi_version": (_i32, []),
    "wx_stream_capture_id": (_i32, [_vp, ctypes.POINTER(ctypes.c_ulonglong)]),
    "wx_partition_workspace_bytes": (_sz, [_i64]),
    "wx_partition_build": (_i32, [_vp, _i32, _i64, _i32, _i32, _i64, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "wx_partition_build_noalloc": (_i32, [_vp, _i32, _i64, _i32, _i32, _i64, _vp, _vp, _vp, _vp, _vp]),
    "wx_partition_noalloc_init": (_i32, []),
    "wx_permute_rows": (_i32, [_vp, _vp, _vp, _i64, _i32, _i64, _i32, _vp]),
    "wx_unpermute_rows": (_i32, [_vp, _vp, _vp, _vp, _i64, _i32, _i64, _i32, _vp]),
    "wx_unpermute_rows_bwd": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i32, _i64, _i32, _vp]),
    "wx_dual_gemm": (_i32, [_vp] * 6 + [_i64] * 6 + [_i32, _i32, _vp]),
    "wx_dual_gemm_add": (_i32, [_vp] * 8 + [_i64] * 6 + [_i32, _i32, _vp]),
    "wx_tiled_bytes": (_sz, [_i64, _i64]),
    "wx_padded_sorted_rows": (_i64, [_i64]),
    "wx_pack_tiled": (_i32, [_vp, _vp, _i64, _i64, _vp]),
    "wx_permute_rows_tiled": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "wx_dual_swiglu_ffn": (_i32, [_vp] * 10 + [_i64] * 4 + [_vp, _vp, _vp]),
    "wx_ffn_fused_workspace_bytes": (_sz, []),
    "wx_dual_swiglu_ffn_fused": (_i32, [_vp] * 12 + [_i64] * 4 + [_vp, _vp, _vp, _vp]),
    "wx_dual_swiglu_gate_up": (_i32, [_vp] * 7 + [_i64] * 4 + [_vp, _vp]),
    "wx_dual_swiglu_gate_up_keep": (_i32, [_vp] * 9 + [_i64] * 4 + [_vp, _vp]),
    "wx_dual_down_proj": (_i32, [_vp] * 5 + [_i64] * 4 + [_vp, _vp, _vp]),
    "wx_dual_down_proj_residual": (_i32, [_vp] * 6 + [_i64] * 4 + [_vp, _vp, _vp]),
    "wx_mrope_apply": (_i32, [_vp] * 6 + [_i64, _i64, _i32, _i32, _i32] + [_c.POINTER(_i64)] * 4
                       + [_c.POINTER(_i32), _i32, _i32, _vp]),
    "wx_mrope_apply_bwd": (_i32, [_vp] * 6 + [_i64, _i64, _i32, _i32, _i32] + [_c.POINTER(_i64)] * 4
                           + [_c.POINTER(_i32), _i32, _i32, _vp]),
    "wx_mrope_apply_positions": (_i32, [_vp] * 6 + [_i64, _i64, _i32, _i32, _i32] + [_c.POINTER(_i64)] * 4
                                 + [_c.POINTER(_i32), _i32, _i32, _i32, _vp]),
    "wx_mrope_table_width": (_i32, [_i32, _c.POINTER(_i32), _i32]),
    "wx_mrope_table": (_i32, [_vp, _vp, _i64, _i64, _i32, _c.POINTER(_i32), _i32, _vp, _vp]),
    "wx_mrope_apply_packed": (_i32, [_vp] * 5 + [_i64, _i64, _i32, _i32, _i32] + [_c.POINTER(_i64)] * 4
                              + [_c.POINTER(_i32), _i32, _i32, _i32, _vp]),
    "wx_qkv_rope_proj": (_i32, [_vp, _vp, _vp, _vp, _i32, _vp, _i64, _i64, _i32, _i32, _i32, _vp]),
    "wx_rope_index_workspace_bytes": (_sz, [_i64, _i64]),
    "wx_rope_index": (_i32, [_vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _i64, _i32, _i64, _i64, _i64, _f32,
                             _vp, _vp, _vp, _vp, _sz, _vp]),
    "wx_rot_pos_emb": (_i32, [_vp, _i32, _vp, _i32, _i64, _i32, _i64, _vp, _vp, _vp]),
    "wx_window_index": (_i32, [_vp, _i32, _i64, _i32, _i32, _i32, _i64, _i64, _vp, _vp, _vp]),
    "wx_rmsnorm_permute_rows_tiled": (_i32, [_vp, _vp, _f32, _vp, _vp, _vp, _i64, _i64, _vp]),
    "wx_unpermute_rows_add": (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "wx_unpermute_rows_add_rmsnorm": (_i32, [_vp, _vp, _vp, _vp, _vp, _f32, _vp, _i64, _i64, _vp]),
    "wx_rmsnorm_permute_rows": (_i32, [_vp, _vp, _f32, _vp, _vp, _i64, _i64, _vp]),
    "wx_rmsnorm_bwd_workspace_bytes": (_sz, [_i64]),
    "wx_unpermute_rows_rmsnorm_bwd": (_i32, [_vp, _vp, _vp, _f32, _vp, _vp, _vp, _vp, _i64, _i64, _vp, _sz, _vp]),
    "wx_moe_block_forward": (_i32, [_vp] * 13 + [_i64] * 4 + [_vp, _vp, _f32, _i32, _vp, _vp]),
    "wx_swiglu_bwd": (_i32, [_vp] * 6 + [_i64, _vp]),
    "wx_swiglu_bwd_tiled": (_i32, [_vp, _vp, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _vp]),
}

_lock = threading.Lock()
_lib = None


class WallxLibraryError(RuntimeError):
    pass


def load():
    """Returns the loaded library; raises WallxLibraryError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise WallxLibraryError(
                    f"{LIB_PATH} is missing: build it with `python wall-x_amd/csrc/build.py` "
                    "(hipcc, gfx950). There is no fallback implementation.")
            lib = ctypes.CDLL(LIB_PATH)
            for name, (res, args) in PROTOTYPES.items():
                fn = getattr(lib, name)  # AttributeError here means header and library disagree
                fn.restype = res
                fn.argtypes = args
            _lib = lib
    return _lib


def check(rc: int, exc=RuntimeError):
    if rc != 0:
        msg = load().wx_last_error_string().decode("utf-8", "replace")
        raise exc(f"wallx_mi355: {msg} (status {rc})")


def call(name: str, *args, exc=RuntimeError):
    check(getattr(load(), name)(*args), exc)


def i64x2(vals):
    """Host int64[2] for the optional per-expert row counts of the FFN entry points; None stays NULL."""
    return None if vals is None else (_i64 * 2)(int(vals[0]), int(vals[1]))


def i64x3(vals):
    return (_i64 * 3)(*[int(v) for v in vals])


def i32x3(vals):
    return (_i32 * 3)(*[int(v) for v in vals])
