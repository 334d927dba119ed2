"""The nine native ops of the reference's ``wallx_csrc`` extension module (csrc/ops.cu:11-21), with the
same names, argument order and ownership rules, implemented on libwallx_mi355.so.

torch is used for allocation and stream lookup only; every computation is a HIP kernel behind the C ABI.
Nothing here falls back to PyTorch math: without the library, or with CPU tensors, calls raise.
"""

import ctypes
import os
import warnings
from typing import List, Optional, Tuple

import torch

from . import _lib
from ._lib import WX_BF16, WX_F16, WX_F32, WX_I32, WX_I64, WX_U8, WX_MROPE_CSRC, WX_MROPE_HF

_DTYPES = {torch.float32: WX_F32, torch.float16: WX_F16, torch.bfloat16: WX_BF16}
_ITYPES = {torch.int32: WX_I32, torch.int64: WX_I64, torch.bool: WX_U8, torch.uint8: WX_U8}

# Channel -> position-plane layouts of the M-RoPE kernels.  "csrc" is the reference's CUDA kernel
# (csrc/rope.cu:104-117), "hf" its PyTorch path (vl.py:763-769).  They differ on 80 of 128 channels for
# mrope_section [16, 24, 24] and coincide only when the three position planes are equal.  The layout is an argument
# of every call (no process-wide switch): rope() / rope_bwd(), the two names of the reference's extension module,
# default to the extension's own layout; the ops that follow the model's PyTorch path pass "hf".
_LAYOUTS = {"hf": WX_MROPE_HF, "csrc": WX_MROPE_CSRC}


def _layout_code(layout: str) -> int:
    try:
        return _LAYOUTS[layout]
    except KeyError:
        raise RuntimeError(f"mrope layout must be 'hf' or 'csrc', got {layout!r}")


# Checked mode.  The kernels report malformed input (expert ids outside the bins, rows whose vision tokens and grids
# do not add up) through a device status word instead of stopping; reading it costs a host synchronisation, which the
# hot path never makes.  With WALLX_MI355_CHECKED=1 in the environment, or set_checked(True), every partition() and
# rope_index() call reads its status word back and raises where the reference's Python path raises.
_checked = os.environ.get("WALLX_MI355_CHECKED", "0") not in ("", "0")


def set_checked(flag: bool) -> None:
    global _checked
    _checked = bool(flag)


def is_checked() -> bool:
    return _checked


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def capture_id(stream: int) -> int:
    """Id of the HIP graph capture `stream` is in, 0 when it is not being captured.  State kept between calls (the
    cached token partition, the shared work buffers) is keyed on it: what is recorded during a capture has not
    executed when the capture ends, and belongs to that graph's replays only."""
    out = ctypes.c_ulonglong(0)  # per call: the library call runs without the interpreter lock
    rc = _lib.load().wx_stream_capture_id(stream, ctypes.byref(out))
    if rc < 0:
        _lib.check(rc)
    return int(out.value) if rc == 1 else 0


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None or t.numel() == 0:
        return None
    return t.data_ptr()


def _need_cuda(name: str, t: torch.Tensor) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")


def _dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise RuntimeError("Wrong activation tensor type.")  # csrc/permute.cu:626


class _DeviceGuard:
    """Makes the tensor's device current for the launch when it is not already."""

    def __init__(self, t: torch.Tensor):
        self.idx = t.device.index
        self.prev = None

    def __enter__(self):
        cur = torch.cuda.current_device()
        if self.idx is not None and self.idx != cur:
            self.prev = cur
            torch.cuda.set_device(self.idx)

    def __exit__(self, *exc):
        if self.prev is not None:
            torch.cuda.set_device(self.prev)


# ----------------------------------------------------------------------------- dual grouped GEMM
def asym_dual_gmm(input_expert0, input_expert1, weight_expert0, weight_expert1, output_expert0,
                  output_expert1, trans_a: bool, trans_b: bool, add_expert0: Optional[torch.Tensor] = None,
                  add_expert1: Optional[torch.Tensor] = None) -> None:
    """csrc/dual_asym_grouped_gemm.cu:308-366.  Writes into the caller's outputs.  add_expert{0,1} (not in the
    reference): contiguous tensors of the outputs' shapes added to the products (they may be the outputs)."""
    ts = (input_expert0, input_expert1, weight_expert0, weight_expert1, output_expert0, output_expert1)
    adds = (add_expert0, add_expert1)
    for add, out in zip(adds, (output_expert0, output_expert1)):
        if add is not None and (add.shape != out.shape or add.dtype != out.dtype or add.device != out.device or
                                not add.is_contiguous()):
            raise RuntimeError("an addend must be a contiguous tensor of its output's shape, dtype and device")
    for t in ts:
        _need_cuda("All tensors", t)
        if t.device != ts[0].device:
            raise RuntimeError("All tensors must be on the same device")
        if t.dtype != torch.bfloat16:
            raise RuntimeError("All tensors must be BFloat16 for this kernel")
    if not (output_expert0.is_contiguous() and output_expert1.is_contiguous()):
        # the reference silently writes a temporary here (csrc/dual_asym_grouped_gemm.cu:335-336); refuse instead
        raise RuntimeError("output tensors must be contiguous")
    a0, a1 = input_expert0.contiguous(), input_expert1.contiguous()
    w0, w1 = weight_expert0.contiguous(), weight_expert1.contiguous()

    def dims(a, w):
        m, k = (a.size(1), a.size(0)) if trans_a else (a.size(0), a.size(1))
        n, kw = (w.size(0), w.size(1)) if trans_b else (w.size(1), w.size(0))
        if k != kw:
            raise RuntimeError(f"inner dimensions disagree: {k} vs {kw}")
        return m, n, k

    m0, n0, k0 = dims(a0, w0)
    m1, n1, k1 = dims(a1, w1)
    if tuple(output_expert0.shape) != (m0, n0) or tuple(output_expert1.shape) != (m1, n1):
        raise RuntimeError("output shape mismatch")
    # Every layout runs on the MFMA kernel: operands stored with K as the slow dimension (trans_a, or weights kept
    # [k, n]) are transposed between LDS and the registers, so no transposed copy is made.
    with _DeviceGuard(a0):
        if add_expert0 is None and add_expert1 is None:
            _lib.call("wx_dual_gemm", _ptr(a0), _ptr(a1), _ptr(w0), _ptr(w1), _ptr(output_expert0),
                      _ptr(output_expert1), m0, n0, k0, m1, n1, k1, int(bool(trans_a)), int(bool(trans_b)),
                      _stream(a0))
        else:
            _lib.call("wx_dual_gemm_add", _ptr(a0), _ptr(a1), _ptr(w0), _ptr(w1), _ptr(output_expert0),
                      _ptr(output_expert1), _ptr(add_expert0), _ptr(add_expert1), m0, n0, k0, m1, n1, k1,
                      int(bool(trans_a)), int(bool(trans_b)), _stream(a0))


def swiglu_bwd(gate: torch.Tensor, up: torch.Tensor, dh: torch.Tensor):
    """(hmid, dgate, dup) of h = silu(gate) * up for the gradient dh, in one pass (bf16, same shapes)."""
    for name, t in (("gate", gate), ("up", up), ("dh", dh)):
        _need_cuda(name, t)
        if t.dtype != torch.bfloat16:
            raise RuntimeError("All tensors must be BFloat16 for this kernel")
    if gate.shape != up.shape or gate.shape != dh.shape:
        raise RuntimeError("gate, up and dh must have one shape")
    gate, up, dh = gate.contiguous(), up.contiguous(), dh.contiguous()
    hm, dg, du = torch.empty_like(gate), torch.empty_like(gate), torch.empty_like(gate)
    with _DeviceGuard(gate):
        _lib.call("wx_swiglu_bwd", _ptr(gate), _ptr(up), _ptr(dh), _ptr(hm), _ptr(dg), _ptr(du), gate.numel(),
                  _stream(gate))
    return hm, dg, du


# ----------------------------------------------------------------------------- permute / unpermute
def partition(indices: torch.Tensor, num_experts: int, num_out_tokens: int = 0,
              workspace: Optional[List[torch.Tensor]] = None, want_sorted: bool = False):
    """Stable partition of expert ids [T] or [T, K] (int32 / int64 / bool, no cast kernel needed).

    Returns (row_id_map int32 [T*K], expert_offsets int32 [E+1], sorted_row_id or None, workspace).
    workspace = [hist scratch, status word]; pass the returned list back in to avoid reallocation.
    Ids outside [0, num_experts) are clamped into range and flagged in the status word (workspace[1], a device
    int32 that stays set until cleared); in checked mode (set_checked / WALLX_MI355_CHECKED=1) the word is cleared
    before and read after every call and such ids raise.
    """
    _need_cuda("indices", indices)
    ids = indices if indices.is_contiguous() else indices.contiguous()
    if ids.dtype not in _ITYPES:
        ids = ids.to(torch.int32)
    T = ids.size(0)
    K = ids.size(1) if ids.dim() == 2 else 1
    n = T * K
    dev = ids.device
    need = _lib.load().wx_partition_workspace_bytes(n)
    if not workspace or workspace[0].numel() < need or workspace[0].device != dev:
        workspace = [torch.empty(need, dtype=torch.uint8, device=dev),
                     torch.zeros(1, dtype=torch.int32, device=dev)]
    elif _checked:
        workspace[1].zero_()  # the status word only ever gets set by the kernels: start each checked call from 0
    row_id_map = torch.empty(n, dtype=torch.int32, device=dev)
    offsets = torch.empty(num_experts + 1, dtype=torch.int32, device=dev)
    sorted_row_id = torch.empty(n, dtype=torch.int32, device=dev) if want_sorted else None
    with _DeviceGuard(ids):
        _lib.call("wx_partition_build", _ptr(ids), _ITYPES[ids.dtype], T, K, int(num_experts),
                  int(num_out_tokens), _ptr(row_id_map), _ptr(sorted_row_id), offsets.data_ptr(),
                  workspace[1].data_ptr(), workspace[0].data_ptr(), workspace[0].numel(), _stream(ids))
    if _checked and n and int(workspace[1].item()):
        raise RuntimeError(f"partition: expert ids outside [0, {int(num_experts)}) (they were clamped into range; "
                           "the grouping does not follow the ids)")
    return row_id_map, offsets, sorted_row_id, workspace


def permute_rows(input: torch.Tensor, row_id_map: torch.Tensor, num_topk: int, num_out: int) -> torch.Tensor:
    out = torch.empty((num_out, input.size(1)), dtype=input.dtype, device=input.device)
    with _DeviceGuard(input):
        _lib.call("wx_permute_rows", _ptr(input), _ptr(out), _ptr(row_id_map), input.size(0), int(num_topk),
                  input.size(1), _dtype_code(input), _stream(input))
    return out


# Expert ids the partition distinguishes.  The reference sorts arbitrary int32 keys with a radix sort;
# MoE expert ids are small, and 256 bins cover every configuration of the model (it has 2 experts).
MAX_EXPERTS = 256


def permute(input: torch.Tensor, indices: torch.Tensor, num_out_tokens: int, workspace: List[torch.Tensor],
            max_expanded_token_num: int) -> Tuple[torch.Tensor, torch.Tensor, List[torch.Tensor]]:
    """csrc/permute.cu:450-630: (permuted [num_out, H], row_id_map int32 [T*K], workspace)."""
    _need_cuda("input", input)
    _need_cuda("indices", indices)
    if input.dim() != 2 or indices.dim() != 2:
        raise RuntimeError("permute expects input [T, H] and indices [T, K]")
    dt = _dtype_code(input)  # raises "Wrong activation tensor type." for unsupported dtypes
    del dt
    if not input.is_contiguous():
        input = input.contiguous()
    T, K = indices.shape
    if K > 128:
        raise RuntimeError("num_topK cannot exceed 128.")  # csrc/permute.cu:394
    row_id_map, _, _, workspace = partition(indices, MAX_EXPERTS, num_out_tokens, workspace)
    num_out = num_out_tokens if num_out_tokens and num_out_tokens > 0 else T * K
    permuted = permute_rows(input, row_id_map, K, num_out)
    return permuted, row_id_map, workspace


def unpermute(input: torch.Tensor, row_id_map: torch.Tensor, prob: torch.Tensor, num_tokens: int,
              num_topK: int) -> torch.Tensor:
    """csrc/permute.cu:638-779.  prob may be an empty tensor (no scaling); ignored when num_topK == 1."""
    _need_cuda("input", input)
    if not input.is_contiguous():
        input = input.contiguous()
    if num_topK > 128:
        raise RuntimeError("num_topK cannot exceed 128.")
    row_id_map = row_id_map.to(device=input.device, dtype=torch.int32).contiguous()
    if row_id_map.numel() < num_tokens * num_topK:
        raise RuntimeError("row_id_map is shorter than num_tokens * num_topK")
    probs = None
    if prob is not None and prob.numel() and num_topK > 1:
        probs = prob.to(device=input.device, dtype=torch.float32).contiguous()
    out = torch.empty((num_tokens, input.size(1)), dtype=input.dtype, device=input.device)
    with _DeviceGuard(input):
        _lib.call("wx_unpermute_rows", _ptr(input), _ptr(out), _ptr(row_id_map), _ptr(probs), int(num_tokens),
                  int(num_topK), input.size(1), _dtype_code(input), _stream(input))
    return out


def unpermute_bwd(input_bwd: torch.Tensor, input_fwd: torch.Tensor, row_id_map: torch.Tensor,
                  prob: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """csrc/permute.cu:781-942: (act_grad [rows of input_fwd, H], prob_grad fp32 [T, K]).

    Rows of act_grad that no token maps to are returned as zeros (the reference leaves them
    uninitialised); prob_grad is zeros when K == 1 (the reference leaves it uninitialised).
    """
    _need_cuda("input_bwd", input_bwd)
    T, K = prob.shape
    input_bwd = input_bwd.contiguous()
    input_fwd = input_fwd.contiguous()
    row_id_map = row_id_map.to(device=input_bwd.device, dtype=torch.int32).contiguous()
    prob = prob.to(device=input_bwd.device, dtype=torch.float32).contiguous()
    act_grad = torch.zeros((input_fwd.size(0), input_bwd.size(1)), dtype=input_bwd.dtype, device=input_bwd.device)
    prob_grad = torch.zeros((T, K), dtype=torch.float32, device=input_bwd.device)
    with _DeviceGuard(input_bwd):
        _lib.call("wx_unpermute_rows_bwd", _ptr(input_bwd), _ptr(input_fwd), _ptr(act_grad), _ptr(prob_grad),
                  _ptr(row_id_map), _ptr(prob), T, K, input_bwd.size(1), _dtype_code(input_bwd),
                  _stream(input_bwd))
    return act_grad, prob_grad


# ----------------------------------------------------------------------------- M-RoPE
def _bhsd_strides(t: torch.Tensor):
    if t.dim() != 4 or t.stride(3) != 1:
        raise RuntimeError("expected a [B, H, S, D] tensor with a contiguous last dimension")
    return _lib.i64x3((t.stride(0), t.stride(1), t.stride(2)))


def _rope_common(fn_name, q_in, k_in, cos, sin, q_out, k_out, mrope_section_doubled, layout):
    for name, t in (("q", q_in), ("k", k_in), ("cos", cos), ("sin", sin), ("q_out", q_out), ("k_out", k_out)):
        _need_cuda(name, t)
    if len(mrope_section_doubled) != 3:
        raise RuntimeError("mrope_section_doubled must have 3 entries")
    B, Hq, S, D = q_in.shape
    Hk = k_in.size(1)
    if tuple(k_in.shape) != (B, Hk, S, D) or tuple(q_out.shape) != tuple(q_in.shape) or \
            tuple(k_out.shape) != tuple(k_in.shape):
        raise RuntimeError("q/k/q_out/k_out shapes are inconsistent")
    if tuple(cos.shape) != (3, B, S, D) or tuple(sin.shape) != (3, B, S, D):
        raise RuntimeError(f"cos/sin must have shape [3, {B}, {S}, {D}]")
    if not (q_in.dtype == k_in.dtype == cos.dtype == sin.dtype == q_out.dtype == k_out.dtype):
        raise RuntimeError("q, k, cos, sin and the outputs must share one dtype")
    cos = cos.contiguous()
    sin = sin.contiguous()
    section = _lib.i32x3([int(v) // 2 for v in mrope_section_doubled])
    with _DeviceGuard(q_in):
        _lib.call(fn_name, _ptr(q_in), _ptr(k_in), _ptr(cos), _ptr(sin), _ptr(q_out), _ptr(k_out), B, S, Hq, Hk,
                  D, _bhsd_strides(q_in), _bhsd_strides(k_in), _bhsd_strides(q_out), _bhsd_strides(k_out),
                  section, _layout_code(layout), _dtype_code(q_in), _stream(q_in))


def rope(q, k, cos, sin, q_out, k_out, mrope_section_doubled, layout: str = "csrc") -> None:
    """csrc/rope.cu:453-509.  q [B,Hq,S,D], k [B,Hkv,S,D] (any batch/head/seq strides), cos/sin [3,B,S,D].
    With the default layout channel d takes plane t for d < 2 s0, h for d < 2 s0 + 2 s1, else w, as the reference's
    kernel does (csrc/rope.cu:104-117); layout="hf" gives apply_multimodal_rotary_pos_emb (vl.py:763-769)."""
    _rope_common("wx_mrope_apply", q, k, cos, sin, q_out, k_out, mrope_section_doubled, layout)


def rope_bwd(grad_q_out, grad_k_out, q, k, cos, sin, grad_q, grad_k, mrope_section_doubled,
             layout: str = "csrc") -> None:
    """csrc/rope.cu:511-571.  q and k are accepted for signature parity; the adjoint does not need them."""
    _rope_common("wx_mrope_apply_bwd", grad_q_out, grad_k_out, cos, sin, grad_q, grad_k, mrope_section_doubled,
                 layout)


def rope_from_positions(q, k, position_ids, inv_freq, q_out, k_out, mrope_section_doubled, backward: bool = False,
                        layout: str = "hf") -> None:
    """M-RoPE with cos/sin evaluated in the kernel (vl.py:679-712 folded into vl.py:731-773): position_ids
    [3, B, S] int64, inv_freq [D/2] fp32.  With backward=True, q/k carry the output gradients and q_out/k_out
    receive the input gradients."""
    for name, t in (("q", q), ("k", k), ("position_ids", position_ids), ("inv_freq", inv_freq), ("q_out", q_out),
                    ("k_out", k_out)):
        _need_cuda(name, t)
    if len(mrope_section_doubled) != 3:
        raise RuntimeError("mrope_section_doubled must have 3 entries")
    B, Hq, S, D = q.shape
    Hk = k.size(1)
    if tuple(k.shape) != (B, Hk, S, D) or tuple(q_out.shape) != tuple(q.shape) or tuple(k_out.shape) != tuple(k.shape):
        raise RuntimeError("q/k/q_out/k_out shapes are inconsistent")
    if tuple(position_ids.shape) != (3, B, S) or position_ids.dtype != torch.int64:
        raise RuntimeError(f"position_ids must be int64 [3, {B}, {S}]")
    if tuple(inv_freq.shape) != (D // 2,) or inv_freq.dtype != torch.float32:
        raise RuntimeError(f"inv_freq must be fp32 [{D // 2}]")
    if not (q.dtype == k.dtype == q_out.dtype == k_out.dtype):
        raise RuntimeError("q, k and the outputs must share one dtype")
    position_ids = position_ids.contiguous()
    inv_freq = inv_freq.contiguous()
    section = _lib.i32x3([int(v) // 2 for v in mrope_section_doubled])
    with _DeviceGuard(q):
        _lib.call("wx_mrope_apply_positions", _ptr(q), _ptr(k), _ptr(position_ids), _ptr(inv_freq), _ptr(q_out),
                  _ptr(k_out), B, S, Hq, Hk, D, _bhsd_strides(q), _bhsd_strides(k), _bhsd_strides(q_out),
                  _bhsd_strides(k_out), section, _layout_code(layout), _dtype_code(q), int(bool(backward)), _stream(q))


def rope_from_table(q, k, table, q_out, k_out, mrope_section_doubled, backward: bool = False,
                    layout: str = "hf") -> None:
    """M-RoPE with cos / sin read from the packed table of mrope_table (int32 [B * S, D / 2] for "hf", [B * S, D] for
    "csrc"; built once per forward for all layers with the same section and layout).  bf16; same results as
    rope_from_positions, bit for bit.  With backward=True, q/k carry the output gradients and q_out/k_out receive
    the input gradients."""
    for name, t in (("q", q), ("k", k), ("table", table), ("q_out", q_out), ("k_out", k_out)):
        _need_cuda(name, t)
    if len(mrope_section_doubled) != 3:
        raise RuntimeError("mrope_section_doubled must have 3 entries")
    B, Hq, S, D = q.shape
    Hk = k.size(1)
    if tuple(k.shape) != (B, Hk, S, D) or tuple(q_out.shape) != tuple(q.shape) or tuple(k_out.shape) != tuple(k.shape):
        raise RuntimeError("q/k/q_out/k_out shapes are inconsistent")
    section = _lib.i32x3([int(v) // 2 for v in mrope_section_doubled])
    width = _table_width(D, section, layout)
    if tuple(table.shape) != (B * S, width) or table.dtype != torch.int32 or not table.is_contiguous():
        raise RuntimeError(f"table must be a contiguous int32 [{B * S}, {width}] tensor from mrope_table with the same "
                           f"mrope_section and layout ({layout!r})")
    if not (q.dtype == k.dtype == q_out.dtype == k_out.dtype == torch.bfloat16):
        raise RuntimeError("All tensors must be BFloat16 for this kernel")
    with _DeviceGuard(q):
        _lib.call("wx_mrope_apply_packed", _ptr(q), _ptr(k), _ptr(table), _ptr(q_out), _ptr(k_out), B, S, Hq, Hk, D,
                  _bhsd_strides(q), _bhsd_strides(k), _bhsd_strides(q_out), _bhsd_strides(k_out), section,
                  _layout_code(layout), _dtype_code(q), int(bool(backward)), _stream(q))


def _table_width(head_dim: int, section_c, layout: str) -> int:
    width = _lib.load().wx_mrope_table_width(int(head_dim), section_c, _layout_code(layout))
    if width < 0:
        _lib.check(width)
    return int(width)


def mrope_table(position_ids: torch.Tensor, inv_freq: torch.Tensor, mrope_section, layout: str = "hf") -> torch.Tensor:
    """Packed rotary table for qkv_rope_proj and rope_from_table: int32 [B * S, W], entry = bf16 cos | bf16 sin << 16
    of position_ids[plane(d)] * inv_freq[d mod D / 2] (vl.py:679-712 rounded to bf16).  position_ids [3, B, S] int64,
    inv_freq [D / 2] fp32, mrope_section the three (un-doubled) section sizes.  W = D / 2 for layout "hf" (channels d
    and d + D / 2 share a position plane and an entry), W = D for "csrc" (one entry per channel)."""
    _need_cuda("position_ids", position_ids)
    _need_cuda("inv_freq", inv_freq)
    if position_ids.dim() != 3 or position_ids.size(0) != 3 or position_ids.dtype != torch.int64:
        raise RuntimeError("position_ids must be int64 [3, B, S]")
    if inv_freq.dim() != 1 or inv_freq.dtype != torch.float32:
        raise RuntimeError("inv_freq must be fp32 [D / 2]")
    if len(mrope_section) != 3:
        raise RuntimeError("mrope_section must have 3 entries")
    _, B, S = position_ids.shape
    half = inv_freq.numel()
    position_ids, inv_freq = position_ids.contiguous(), inv_freq.contiguous()
    section = _lib.i32x3([int(v) for v in mrope_section])
    table = torch.empty((B * S, _table_width(2 * half, section, layout)), dtype=torch.int32, device=position_ids.device)
    with _DeviceGuard(position_ids):
        _lib.call("wx_mrope_table", _ptr(position_ids), _ptr(inv_freq), B, S, 2 * half, section, _layout_code(layout),
                  _ptr(table), _stream(position_ids))
    return table


def qkv_rope_proj(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], table: torch.Tensor,
                  n_q_heads: int, n_kv_heads: int, head_dim: int = 128, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [..., hidden] @ weight^T + bias with M-RoPE applied to the q and k heads in the GEMM's epilogue
    (vl.py:955-964 in one launch).  weight [(n_q + 2 n_kv) * head_dim, hidden] = q, k, v weights stacked, bias likewise
    or None, table from mrope_table (one row per row of x; its width says whether channels d and d + D / 2 share an
    entry, so either channel layout is served).  Returns [..., (n_q + 2 n_kv) * head_dim]: columns [0, n_q D) are the
    rotated q heads, the next n_kv D the rotated k heads, the last n_kv D the v heads."""
    for name, t in (("x", x), ("weight", weight), ("table", table)):
        _need_cuda(name, t)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or (bias is not None and bias.dtype != torch.bfloat16):
        raise RuntimeError("All tensors must be BFloat16 for this kernel")
    hidden = x.shape[-1]
    n = (n_q_heads + 2 * n_kv_heads) * head_dim
    if weight.dim() != 2 or tuple(weight.shape) != (n, hidden):
        raise RuntimeError(f"weight must be [{n}, {hidden}] (q, k and v projection weights stacked)")
    if bias is not None and tuple(bias.shape) != (n,):
        raise RuntimeError(f"bias must be [{n}]")
    x2 = x.reshape(-1, hidden)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    T = x2.size(0)
    if table.dtype != torch.int32 or table.dim() != 2 or table.size(0) != T or \
            table.size(1) not in (head_dim // 2, head_dim):
        raise RuntimeError(f"table must be int32 [{T}, {head_dim // 2}] or [{T}, {head_dim}] (mrope_table of the same "
                           "tokens)")
    weight = weight.contiguous()
    table = table.contiguous()
    bias = None if bias is None else bias.contiguous()
    if out is None or out.dtype != torch.bfloat16 or out.numel() != T * n or not out.is_contiguous() or out.device != x.device:
        out = torch.empty((T, n), dtype=torch.bfloat16, device=x.device)
    with _DeviceGuard(x2):
        _lib.call("wx_qkv_rope_proj", _ptr(x2), _ptr(weight), _ptr(bias), _ptr(table), int(table.size(1)), _ptr(out), T,
                  hidden, int(n_q_heads), int(n_kv_heads), int(head_dim), _stream(x2))
    return out.view(*x.shape[:-1], n)


# ----------------------------------------------------------------------------- index builders
def rope_index(input_ids, image_grid_thw, video_grid_thw, second_per_grid_ts, attention_mask,
               spatial_merge_size: int, image_token_id: int, video_token_id: int, vision_start_token_id: int,
               tokens_per_second: float, return_status: bool = False):
    """csrc/rope_index.cu:464-569 with the PyTorch path's semantics (act.py:929-1149).

    Returns (position_ids int64 [3, B, S], mrope_deltas int64 [B, 1]).
    """
    if input_ids is None:
        raise RuntimeError("input_ids is required")
    _need_cuda("input_ids", input_ids)
    dev = input_ids.device

    def as_i64(t):
        return None if t is None else t.to(device=dev, dtype=torch.int64).contiguous()

    ids = as_i64(input_ids)
    B, S = ids.shape
    mask = as_i64(attention_mask)
    ig, vg = as_i64(image_grid_thw), as_i64(video_grid_thw)
    spg = None if second_per_grid_ts is None else second_per_grid_ts.to(device=dev, dtype=torch.float32).contiguous()
    pos = torch.empty((3, B, S), dtype=torch.int64, device=dev)
    deltas = torch.empty((B, 1), dtype=torch.int64, device=dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    ws_bytes = _lib.load().wx_rope_index_workspace_bytes(B, S)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    with _DeviceGuard(ids):
        _lib.call("wx_rope_index", _ptr(ids), _ptr(mask), None if ig is None else ig.data_ptr(),
                  0 if ig is None else ig.size(0), None if vg is None else vg.data_ptr(),
                  0 if vg is None else vg.size(0), _ptr(spg), B, S, int(spatial_merge_size), int(image_token_id),
                  int(video_token_id), int(vision_start_token_id), float(tokens_per_second), _ptr(pos),
                  _ptr(deltas), status.data_ptr(), ws.data_ptr(), ws_bytes, _stream(ids))
    if _checked and int(status.item()):
        # the Python path raises on such rows (list.index / grid indexing, act.py:1013-1045)
        raise ValueError("rope_index: a row's vision tokens, <vision_start> markers and grids do not add up "
                         "(or a row is fully masked)")
    if return_status:
        return pos, deltas, status
    return pos, deltas


def _host_grid(grid_thw: torch.Tensor, grid_thw_host):
    """grid_thw as a host list of (t, h, w); copies device -> host (one sync) unless a host copy is given."""
    if grid_thw_host is not None:
        src = grid_thw_host
    else:
        src = grid_thw
    return [tuple(int(v) for v in row) for row in src.cpu().tolist()]


def rot_pos_emb(inv_freq: torch.Tensor, grid_thw: torch.Tensor, spatial_merge_size: int,
                grid_thw_host: Optional[torch.Tensor] = None, return_ids: bool = False):
    """csrc/rot_pos.cu:187-312: fp32 [sum t*h*w, 2*len(inv_freq)].

    The output size depends on grid_thw's values; pass grid_thw_host (the CPU copy the processor produced)
    to avoid the device -> host read the reference also performs.
    """
    _need_cuda("inv_freq", inv_freq)
    _need_cuda("grid_thw", grid_thw)
    if inv_freq.dtype != torch.float32:
        raise RuntimeError("inv_freq must be float32")
    if grid_thw.dtype not in (torch.int32, torch.int64):
        raise RuntimeError("grid_thw must be int32 or int64")
    grid = grid_thw.contiguous()
    inv = inv_freq.contiguous()
    rows = _host_grid(grid, grid_thw_host)
    total = sum(t * h * w for t, h, w in rows)
    F = inv.numel()
    table = torch.empty((total, 2 * F), dtype=torch.float32, device=inv.device)
    ids = torch.empty((total, 2), dtype=torch.int64, device=inv.device) if return_ids else None
    with _DeviceGuard(inv):
        _lib.call("wx_rot_pos_emb", _ptr(inv), F, _ptr(grid), _ITYPES[grid.dtype], grid.size(0),
                  int(spatial_merge_size), total, _ptr(table), _ptr(ids), _stream(inv))
    return (table, ids) if return_ids else table


def get_window_index(grid_thw: torch.Tensor, spatial_merge_size: int, vit_merger_window_size: int,
                     patch_size: int, spatial_merge_unit: int, grid_thw_host: Optional[torch.Tensor] = None):
    """csrc/window_index.cu:208-286: (window_index int32 [N], cu_window_seqlens int32 [W + 1])."""
    _need_cuda("grid_thw", grid_thw)
    if grid_thw.dim() != 2 or grid_thw.size(1) != 3:
        raise RuntimeError("grid_thw must have shape [num_grids, 3]")
    if grid_thw.dtype != torch.int32:
        raise RuntimeError("grid_thw must be int32")  # csrc/window_index.cu:217
    del patch_size  # part of the reference signature; the window size arrives already divided by it
    grid = grid_thw.contiguous()
    dev = grid.device
    if grid.size(0) == 0:  # csrc/window_index.cu:220-225
        return torch.empty(0, dtype=torch.int32, device=dev), torch.zeros(1, dtype=torch.int32, device=dev)
    rows = _host_grid(grid, grid_thw_host)
    m, ws = int(spatial_merge_size), int(vit_merger_window_size)
    n_tok = sum(t * (h // m) * (w // m) for t, h, w in rows)
    n_win = sum(t * (-(-(h // m) // ws)) * (-(-(w // m) // ws)) for t, h, w in rows)
    if n_tok == 0 or n_win == 0:  # csrc/window_index.cu:253-258
        return torch.empty(0, dtype=torch.int32, device=dev), torch.zeros(1, dtype=torch.int32, device=dev)
    window_index = torch.empty(n_tok, dtype=torch.int32, device=dev)
    cu = torch.empty(n_win + 1, dtype=torch.int32, device=dev)
    with _DeviceGuard(grid):
        _lib.call("wx_window_index", _ptr(grid), WX_I32, grid.size(0), m, ws, int(spatial_merge_unit), n_tok,
                  n_win, _ptr(window_index), _ptr(cu), _stream(grid))
    return window_index, cu


# ----------------------------------------------------------------------------- fused dual-expert FFN
import weakref

_packed_cache = {}  # id(weight) -> (weakref to weight, (data_ptr, version, shape, device), packed tensor)


def padded_sorted_rows(num_tokens: int) -> int:
    """Rows of the expert-sorted space once each expert's range starts at a multiple of 256."""
    return int(_lib.load().wx_padded_sorted_rows(int(num_tokens)))


def invalidate_packed(w: Optional[torch.Tensor] = None) -> None:
    """Drops the cached K-tiled copy of `w` (of every weight when w is None).  Call it after writing a weight in a
    way torch's version counter does not see -- `w.data.copy_(...)`, `w.data.normal_()`, a write through another
    view of `.data` -- before the next forward that does not track gradients."""
    if w is None:
        _packed_cache.clear()
    else:
        _packed_cache.pop(id(w), None)
    for hook in _invalidate_hooks:  # holders of objects built from packed copies (moe's per-weight-set cache)
        hook(w)


_invalidate_hooks = []


def pack_weight(w: torch.Tensor, cache: bool = True) -> torch.Tensor:
    """nn.Linear weight [out, in] (bf16, CUDA) -> the K-tiled layout the MFMA kernels read (flat bf16 tensor).

    Packed copies are cached per weight tensor, keyed on its storage address, shape and version counter, so an
    in-place update through the tensor itself (an optimizer step, `copy_`, `load_state_dict`) or a re-assigned
    `.data` repacks.  Writes through `.data` do not move the version counter: callers whose weights train pass
    cache=False (the MoE block does, on its autograd path: tens of microseconds beside the GEMMs the weights feed
    and their backward), and frozen weights written that way need invalidate_packed()."""
    _need_cuda("weight", w)
    if w.dtype != torch.bfloat16 or w.dim() != 2:
        raise RuntimeError("expert weights must be 2-D BFloat16 tensors")
    key = id(w)
    if w.is_inference():
        cache = False  # a tensor made under torch.inference_mode() has no version counter to check a cached copy against
    if not cache:
        _packed_cache.pop(key, None)
    state = (w.data_ptr(), None if not cache else w._version, tuple(w.shape), w.device)
    if cache:
        hit = _packed_cache.get(key)
        if hit is not None and hit[0]() is w and hit[1] == state:
            return hit[2]
    src = w.detach().contiguous()
    rows, cols = src.shape
    nbytes = _lib.load().wx_tiled_bytes(rows, cols)
    packed = torch.empty(nbytes // 2, dtype=torch.bfloat16, device=w.device)
    with _DeviceGuard(src):
        _lib.call("wx_pack_tiled", _ptr(src), packed.data_ptr(), rows, cols, _stream(src))
    if cache:
        _packed_cache[key] = (weakref.ref(w, lambda _r, k=key: _packed_cache.pop(k, None)), state, packed)
    return packed


def permute_rows_tiled(x: torch.Tensor, row_id_map: Optional[torch.Tensor], expert_offsets: torch.Tensor,
                       out: Optional[torch.Tensor] = None, sorted_row_id: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [T, H] bf16 -> K-tiled, expert-padded activation matrix for dual_swiglu_ffn (flat bf16 tensor).

    With sorted_row_id (partition(..., want_sorted=True)) the rows are gathered block by block, the faster form."""
    _need_cuda("x", x)
    if x.dtype != torch.bfloat16:
        raise RuntimeError("All tensors must be BFloat16 for this kernel")
    x = x.contiguous()
    T, H = x.shape
    need = _lib.load().wx_tiled_bytes(padded_sorted_rows(T), H) // 2
    if out is None or out.numel() < need or out.dtype != torch.bfloat16 or out.device != x.device:
        out = torch.empty(need, dtype=torch.bfloat16, device=x.device)
    with _DeviceGuard(x):
        _lib.call("wx_permute_rows_tiled", _ptr(x), out.data_ptr(), _ptr(row_id_map), _ptr(sorted_row_id),
                  expert_offsets.data_ptr(), T, H, _stream(x))
    return out


def rmsnorm_permute_rows_tiled(x: torch.Tensor, weight: torch.Tensor, eps: float, expert_offsets: torch.Tensor,
                               sorted_row_id: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm(x) * weight written straight into the K-tiled, expert-padded activation matrix (one pass)."""
    _need_cuda("x", x)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise RuntimeError("All tensors must be BFloat16 for this kernel")
    x, weight = x.contiguous(), weight.contiguous()
    T, H = x.shape
    if weight.numel() != H:
        raise RuntimeError("weight size must equal the hidden size")
    need = _lib.load().wx_tiled_bytes(padded_sorted_rows(T), H) // 2
    if out is None or out.numel() < need or out.dtype != torch.bfloat16 or out.device != x.device:
        out = torch.empty(need, dtype=torch.bfloat16, device=x.device)
    with _DeviceGuard(x):
        _lib.call("wx_rmsnorm_permute_rows_tiled", _ptr(x), _ptr(weight), float(eps), out.data_ptr(),
                  _ptr(sorted_row_id), expert_offsets.data_ptr(), T, H, _stream(x))
    return out


def unpermute_add(y_sorted: torch.Tensor, residual: torch.Tensor, row_id_map: torch.Tensor) -> torch.Tensor:
    """residual + y_sorted[row_id_map] in one pass (topK 1, bf16)."""
    _need_cuda("y_sorted", y_sorted)
    if y_sorted.dtype != torch.bfloat16 or residual.dtype != torch.bfloat16:
        raise RuntimeError("All tensors must be BFloat16 for this kernel")
    y_sorted, residual = y_sorted.contiguous(), residual.contiguous()
    T, H = residual.shape
    if y_sorted.shape[1] != H or row_id_map.numel() < T:
        raise RuntimeError("shape mismatch between residual, sorted rows and row_id_map")
    out = torch.empty_like(residual)
    with _DeviceGuard(residual):
        _lib.call("wx_unpermute_rows_add", _ptr(y_sorted), _ptr(residual), _ptr(out), _ptr(row_id_map), T, H,
                  _stream(residual))
    return out


def unpermute_add_rmsnorm(y_sorted: torch.Tensor, residual: torch.Tensor, row_id_map: torch.Tensor,
                          weight: torch.Tensor, eps: float):
    """(residual + y_sorted[row_id_map], rmsnorm of that sum with `weight`) in one pass (topK 1, bf16): the layer's
    closing residual add (act.py:265) and the next layer's input_layernorm (act.py:240) or the final norm."""
    _need_cuda("y_sorted", y_sorted)
    if y_sorted.dtype != torch.bfloat16 or residual.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise RuntimeError("All tensors must be BFloat16 for this kernel")
    y_sorted, residual, weight = y_sorted.contiguous(), residual.contiguous(), weight.contiguous()
    T, H = residual.shape
    if y_sorted.shape[1] != H or row_id_map.numel() < T or weight.numel() != H:
        raise RuntimeError("shape mismatch between residual, sorted rows, weight and row_id_map")
    out, normed = torch.empty_like(residual), torch.empty_like(residual)
    with _DeviceGuard(residual):
        _lib.call("wx_unpermute_rows_add_rmsnorm", _ptr(y_sorted), _ptr(residual), _ptr(out), _ptr(normed),
                  _ptr(weight), float(eps), _ptr(row_id_map), T, H, _stream(residual))
    return out, normed


def rmsnorm_permute_rows(x: torch.Tensor, weight: torch.Tensor, eps: float, sorted_row_id: torch.Tensor) -> torch.Tensor:
    """weight * rmsnorm(x)[sorted_row_id]: the normed rows in expert-sorted order, row-major (one pass)."""
    _need_cuda("x", x)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise RuntimeError("All tensors must be BFloat16 for this kernel")
    x, weight = x.contiguous(), weight.contiguous()
    T, H = x.shape
    if weight.numel() != H or sorted_row_id.numel() < T or sorted_row_id.dtype != torch.int32:
        raise RuntimeError("weight size must equal the hidden size, sorted_row_id must be int32 with one entry per row")
    out = torch.empty_like(x)
    with _DeviceGuard(x):
        _lib.call("wx_rmsnorm_permute_rows", _ptr(x), _ptr(weight), float(eps), _ptr(out), _ptr(sorted_row_id), T, H,
                  _stream(x))
    return out


def unpermute_rmsnorm_bwd(grad_sorted: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, eps: float,
                          row_id_map: torch.Tensor, add: Optional[torch.Tensor] = None):
    """Backward of `permute(weight * rmsnorm(x))` for the gradient of the sorted rows, in one pass (topK 1, bf16):
    returns (grad_x [T, H] -- with `add`, a [T, H] gradient arriving along the residual branch, summed in -- and
    grad_weight [H])."""
    _need_cuda("grad_sorted", grad_sorted)
    for t in (grad_sorted, x, weight) + ((add,) if add is not None else ()):
        if t.dtype != torch.bfloat16:
            raise RuntimeError("All tensors must be BFloat16 for this kernel")
    grad_sorted, x, weight = grad_sorted.contiguous(), x.contiguous(), weight.contiguous()
    T, H = x.shape
    if grad_sorted.shape[1] != H or row_id_map.numel() < T or weight.numel() != H or \
            (add is not None and tuple(add.shape) != (T, H)):
        raise RuntimeError("shape mismatch between the sorted gradient, x, weight, add and row_id_map")
    add = None if add is None else add.contiguous()
    gx = torch.empty_like(x)
    gw = torch.empty(H, dtype=torch.bfloat16, device=x.device)
    nbytes = _lib.load().wx_rmsnorm_bwd_workspace_bytes(H)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    with _DeviceGuard(x):
        _lib.call("wx_unpermute_rows_rmsnorm_bwd", _ptr(grad_sorted), _ptr(x), _ptr(weight), float(eps), _ptr(add),
                  _ptr(gx), _ptr(gw), _ptr(row_id_map), T, H, ws.data_ptr(), nbytes, _stream(x))
    return gx, gw


def dual_swiglu_ffn_packed(x_tiled: torch.Tensor, num_rows: int, expert_offsets: torch.Tensor, packed, dims,
                           hmid: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                           host_rows=None, out_row_id: Optional[torch.Tensor] = None,
                           residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """dual_swiglu_ffn on weights that are already K-tiled: packed = (gate0, up0, down0, gate1, up1, down1) from
    pack_weight, dims = (hidden, inter0, inter1).  residual (with out_row_id): a [num_rows, hidden] tensor in token
    order added to the result in the down launch's stores."""
    _need_cuda("x_tiled", x_tiled)
    H, I0, I1 = (int(v) for v in dims)
    lib = _lib.load()
    want = [lib.wx_tiled_bytes(I0, H), lib.wx_tiled_bytes(I0, H), lib.wx_tiled_bytes(H, I0),
            lib.wx_tiled_bytes(I1, H), lib.wx_tiled_bytes(I1, H), lib.wx_tiled_bytes(H, I1)]
    if len(packed) != 6:
        raise RuntimeError("packed must hold gate, up and down of both experts")
    for t, nbytes in zip(packed, want):
        _need_cuda("packed weight", t)
        if t.dtype != torch.bfloat16 or t.numel() * 2 < nbytes or t.device != x_tiled.device:
            raise RuntimeError("packed expert weights do not match (hidden, inter0, inter1)")
    if expert_offsets.dtype != torch.int32 or expert_offsets.numel() < 3 or not expert_offsets.is_cuda:
        raise RuntimeError("expert_offsets must be an int32 CUDA tensor with 3 entries")
    if out_row_id is not None and (out_row_id.dtype != torch.int32 or not out_row_id.is_cuda or
                                   out_row_id.numel() < num_rows):
        raise RuntimeError("out_row_id must be an int32 CUDA tensor with one entry per row")
    dev = x_tiled.device
    need = padded_sorted_rows(num_rows) * max(I0, I1)
    if hmid is None or hmid.numel() < need or hmid.dtype != torch.bfloat16:
        hmid = torch.empty(need, dtype=torch.bfloat16, device=dev)
    if out is None:
        out = torch.empty((num_rows, H), dtype=torch.bfloat16, device=dev)
    if residual is not None:
        _check_residual(residual, num_rows, H, dev, out_row_id)
    with _DeviceGuard(x_tiled):
        if residual is not None and num_rows:
            _lib.call("wx_dual_swiglu_gate_up", x_tiled.data_ptr(), hmid.data_ptr(), expert_offsets.data_ptr(),
                      _ptr(packed[0]), _ptr(packed[1]), _ptr(packed[3]), _ptr(packed[4]), int(num_rows), H, I0, I1,
                      _lib.i64x2(host_rows), _stream(x_tiled))
            _lib.call("wx_dual_down_proj_residual", hmid.data_ptr(), _ptr(out), residual.data_ptr(),
                      expert_offsets.data_ptr(), _ptr(packed[2]), _ptr(packed[5]), int(num_rows), H, I0, I1,
                      _lib.i64x2(host_rows), _ptr(out_row_id), _stream(x_tiled))
        else:
            _lib.call("wx_dual_swiglu_ffn", x_tiled.data_ptr(), _ptr(out), expert_offsets.data_ptr(), _ptr(packed[0]),
                      _ptr(packed[1]), _ptr(packed[2]), _ptr(packed[3]), _ptr(packed[4]), _ptr(packed[5]),
                      hmid.data_ptr(), int(num_rows), H, I0, I1, _lib.i64x2(host_rows), _ptr(out_row_id),
                      _stream(x_tiled))
    return out


def _check_residual(residual, num_rows, hidden, dev, out_row_id) -> None:
    if out_row_id is None:
        raise RuntimeError("a residual is added in token order: it needs out_row_id")
    if residual.dtype != torch.bfloat16 or tuple(residual.shape) != (num_rows, hidden) or residual.device != dev or \
            not residual.is_contiguous():
        raise RuntimeError("residual must be a contiguous [num_rows, hidden] BFloat16 tensor on the activations' device")


class HostRows:
    """The partition's expert_offsets on their way to the host without a synchronisation: an asynchronous copy into
    pinned memory, queued behind the partition on its stream, and an event behind the copy.  `ready()` answers None
    until the event has completed and the per-expert row counts as _lib.i64x2 afterwards, so the layers of a forward
    that are queued after the copy has landed hand the counts to the GEMM entry points and get one dispatch each
    instead of one per tile shape (act.py:1274-1283 gives the reference's caller the same numbers on the host)."""

    __slots__ = ("pinned", "event", "rows", "num_tokens")

    def __init__(self, expert_offsets: torch.Tensor, num_tokens: int):
        self.pinned = torch.empty(3, dtype=torch.int32, pin_memory=True)
        self.pinned.copy_(expert_offsets[:3], non_blocking=True)
        self.event = torch.cuda.Event()
        self.event.record(torch.cuda.current_stream(expert_offsets.device))
        self.rows = None
        self.num_tokens = num_tokens

    def ready(self):
        if self.rows is None:
            if self.event is None or not self.event.query():
                return None
            o = self.pinned.tolist()
            self.event = None
            counts = (o[1] - o[0], o[2] - o[1])
            if min(counts) < 0 or sum(counts) != self.num_tokens:
                return None  # rows were dropped (num_out_tokens) or the offsets are not a two-expert split
            self.rows = _lib.i64x2(counts)
        return self.rows


# The block forward's permute and two GEMMs as one launch where the shape allows it (wx_dual_swiglu_ffn_fused: a
# denoise step's few thousand tokens); off: always the separate launches.  WALLX_MI355_ONE_LAUNCH_FFN=0 starts with it off.
_one_launch_ffn = os.environ.get("WALLX_MI355_ONE_LAUNCH_FFN", "1") != "0"


def set_one_launch_ffn(flag: bool) -> bool:
    """Switches the one-launch form of the block forward on or off; returns the previous setting.  Results are
    bit-identical either way."""
    global _one_launch_ffn
    old, _one_launch_ffn = _one_launch_ffn, bool(flag)
    return old

_ffn_scratch = {}  # (device index, stream handle, capturing) -> (tiled activations, intermediate, capture id, counters)


def _ffn_buffers(device: torch.device, stream: int, x_elems: int, h_elems: int, cap: Optional[int] = None):
    """The tiled-activation and intermediate buffers of the block forward, one pair per device and stream: the
    layers of a model run one after the other on a stream, so they can all work in the same two buffers (a pair per
    block would hold 0.45 GB per layer at 29 184 tokens).  Calls that overlap on one stream's pair from two threads
    race, like any two launches writing one buffer.  Under HIP graph capture the pair belongs to that capture (its
    memory comes from the graph's pool and its replays write it): eager calls never share it, and a later capture on
    the same stream replaces it.  With them comes the zeroed counter workspace of the one-launch FFN
    (wx_dual_swiglu_ffn_fused), which every launch leaves zero again."""
    if cap is None:
        cap = capture_id(stream)
    key = (device.index, stream, cap != 0)
    hit = _ffn_scratch.get(key)
    if hit is not None and hit[2] != cap:
        hit = None  # another capture's pair
    if hit is None or hit[0].numel() < x_elems or hit[1].numel() < h_elems:
        if hit is not None:
            x_elems, h_elems = max(x_elems, hit[0].numel()), max(h_elems, hit[1].numel())
        counters = hit[3] if hit is not None and hit[2] == cap else \
            torch.zeros(_lib.load().wx_ffn_fused_workspace_bytes() // 4 + 1, dtype=torch.int32, device=device)
        hit = (torch.empty(x_elems, dtype=torch.bfloat16, device=device),
               torch.empty(h_elems, dtype=torch.bfloat16, device=device), cap, counters)
        _ffn_scratch[key] = hit
    return hit[0], hit[1], cap, hit[3]


def release_ffn_buffers() -> None:
    """Drops the buffers _ffn_buffers keeps (they come back, sized for the next call, when needed)."""
    _ffn_scratch.clear()


class PackedExperts:
    """The six K-tiled projection weights of a two-expert block, checked once, with their addresses ready for the
    launches: what packed_block_forward needs so that a call is two or three library calls and one allocation."""

    __slots__ = ("tensors", "ptrs", "hidden", "inter0", "inter1", "device", "_sizes")

    def __init__(self, packed, dims):
        H, I0, I1 = (int(v) for v in dims)
        lib = _lib.load()
        want = [lib.wx_tiled_bytes(I0, H), lib.wx_tiled_bytes(I0, H), lib.wx_tiled_bytes(H, I0),
                lib.wx_tiled_bytes(I1, H), lib.wx_tiled_bytes(I1, H), lib.wx_tiled_bytes(H, I1)]
        packed = list(packed)
        if len(packed) != 6:
            raise RuntimeError("packed must hold gate, up and down of both experts")
        for t, nbytes in zip(packed, want):
            _need_cuda("packed weight", t)
            if t.dtype != torch.bfloat16 or t.numel() * 2 < nbytes or t.device != packed[0].device or \
                    not t.is_contiguous():
                raise RuntimeError("packed expert weights do not match (hidden, inter0, inter1)")
        self.tensors = packed
        self.ptrs = tuple(_ptr(t) for t in packed)
        self.hidden, self.inter0, self.inter1 = H, I0, I1
        self.device = packed[0].device
        self._sizes = {}

    def sizes(self, num_rows: int):
        """(elements of the tiled activation matrix, elements of the intermediate) for num_rows tokens."""
        hit = self._sizes.get(num_rows)
        if hit is None:
            pad = padded_sorted_rows(num_rows)
            hit = (_lib.load().wx_tiled_bytes(pad, self.hidden) // 2, pad * max(self.inter0, self.inter1))
            if len(self._sizes) >= 64:
                self._sizes.clear()
            self._sizes[num_rows] = hit
        return hit


def packed_block_forward(experts: PackedExperts, x: torch.Tensor, row_id_map: torch.Tensor,
                         sorted_row_id: torch.Tensor, expert_offsets: torch.Tensor, host_rows_c=None,
                         pre_norm=None, residual: bool = False, rows_when_ready=None,
                         stream: Optional[int] = None, capture: Optional[int] = None) -> torch.Tensor:
    """One block forward on packed weights, in token order: [RMSNorm ->] permute -> gate/up + SwiGLU -> down with
    the unpermute [and the residual add, + x] in its stores.  x [T, hidden] bf16; the three routing tensors are the partition's
    (int32, on x's device); host_rows_c is None or _lib.i64x2((rows of expert 0, rows of expert 1)).  Without it,
    `rows_when_ready` (a callable returning such a pair or None: the partition's own read-back of expert_offsets, see
    HostRows) is asked outside HIP graph captures; a capture always records the launches that decide on the device.
    The work buffers are shared per stream (see _ffn_buffers); the result is a new tensor.  stream / capture: x's
    device's current stream handle and its capture id, when the caller has them already."""
    dev = x.device
    if dev != experts.device or x.dtype != torch.bfloat16 or x.dim() != 2 or x.shape[1] != experts.hidden:
        raise RuntimeError("x must be a [tokens, hidden] BFloat16 tensor on the device of the packed weights")
    if not x.is_contiguous():
        x = x.contiguous()
    T = x.shape[0]
    for t in (row_id_map, sorted_row_id):
        if t.dtype != torch.int32 or t.device != dev or t.numel() < T:
            raise RuntimeError("row_id_map / sorted_row_id must be int32 tensors on x's device, one entry per token")
    if expert_offsets.dtype != torch.int32 or expert_offsets.device != dev or expert_offsets.numel() < 3:
        raise RuntimeError("expert_offsets must be an int32 CUDA tensor with 3 entries")
    out = torch.empty_like(x)
    if T == 0:
        return out
    lib = _lib.load()
    if stream is None:
        stream = torch.cuda.current_stream(dev).cuda_stream
    x_elems, h_elems = experts.sizes(T)
    x_tiled, hmid, cap, counters = _ffn_buffers(dev, stream, x_elems, h_elems, capture)
    if host_rows_c is None and rows_when_ready is not None and cap == 0:
        host_rows_c = rows_when_ready()
    H, I0, I1 = experts.hidden, experts.inter0, experts.inter1
    norm_ptr, eps = None, 0.0
    if pre_norm is not None:
        weight, eps = pre_norm
        if weight.dtype != torch.bfloat16 or weight.numel() != H or weight.device != dev or \
                not weight.is_contiguous():
            raise RuntimeError("the norm weight must be a contiguous BFloat16 tensor of the hidden size")
        norm_ptr = weight.data_ptr()
    with _DeviceGuard(x):  # one library call: [RMSNorm +] permute, gate/up, down with the unpermute [and the residual]
        _lib.check(lib.wx_moe_block_forward(x.data_ptr(), out.data_ptr(), row_id_map.data_ptr(),
                                            sorted_row_id.data_ptr(), expert_offsets.data_ptr(), *experts.ptrs,
                                            x_tiled.data_ptr(), hmid.data_ptr(), T, H, I0, I1, host_rows_c, norm_ptr,
                                            float(eps), int(bool(residual)),
                                            counters.data_ptr() if _one_launch_ffn else None, stream))
    if _checked and _one_launch_ffn and cap == 0 and int(counters[-1].item()):
        counters.zero_()
        raise RuntimeError("packed_block_forward: a wait inside the one-launch FFN ran into its bound (the result is "
                           "undefined); native.set_one_launch_ffn(False) runs the separate launches")
    return out


def dual_swiglu_ffn_keep(x_tiled: torch.Tensor, num_rows: int, expert_offsets: torch.Tensor, weights,
                         hmid: Optional[torch.Tensor] = None, host_rows=None,
                         out_row_id: Optional[torch.Tensor] = None, frozen=None,
                         residual: Optional[torch.Tensor] = None):
    """dual_swiglu_ffn for a forward pass whose backward follows: the gate / up launch also stores the two
    projections (K-tiled, the intermediate's geometry) so the backward need not run them again.  The weights are
    packed afresh (they train), except those flagged in `frozen` (six booleans in the order gate0, up0, down0, gate1,
    up1, down1), whose packed copies are cached like an inference forward's.  Returns (out, gate_keep, up_keep, hmid)."""
    _need_cuda("x_tiled", x_tiled)
    (g0, u0, d0), (g1, u1, d1) = weights
    H, I0, I1 = g0.size(1), g0.size(0), g1.size(0)
    cached = tuple(frozen) if frozen is not None else (False,) * 6
    packed = [pack_weight(w, cache=c) for w, c in zip((g0, u0, d0, g1, u1, d1), cached)]
    dev = x_tiled.device
    need = padded_sorted_rows(num_rows) * max(I0, I1)
    if hmid is None or hmid.numel() < need or hmid.dtype != torch.bfloat16:
        hmid = torch.empty(need, dtype=torch.bfloat16, device=dev)
    gate_keep = torch.empty(need, dtype=torch.bfloat16, device=dev)
    up_keep = torch.empty(need, dtype=torch.bfloat16, device=dev)
    out = torch.empty((num_rows, H), dtype=torch.bfloat16, device=dev)
    if num_rows == 0:
        return out, gate_keep, up_keep, hmid
    if residual is not None:
        _check_residual(residual, num_rows, H, dev, out_row_id)
    with _DeviceGuard(x_tiled):
        _lib.call("wx_dual_swiglu_gate_up_keep", x_tiled.data_ptr(), hmid.data_ptr(), gate_keep.data_ptr(),
                  up_keep.data_ptr(), expert_offsets.data_ptr(), _ptr(packed[0]), _ptr(packed[1]), _ptr(packed[3]),
                  _ptr(packed[4]), int(num_rows), H, I0, I1, _lib.i64x2(host_rows), _stream(x_tiled))
        if residual is not None:
            _lib.call("wx_dual_down_proj_residual", hmid.data_ptr(), _ptr(out), residual.data_ptr(),
                      expert_offsets.data_ptr(), _ptr(packed[2]), _ptr(packed[5]), int(num_rows), H, I0, I1,
                      _lib.i64x2(host_rows), _ptr(out_row_id), _stream(x_tiled))
        else:
            _lib.call("wx_dual_down_proj", hmid.data_ptr(), _ptr(out), expert_offsets.data_ptr(), _ptr(packed[2]),
                      _ptr(packed[5]), int(num_rows), H, I0, I1, _lib.i64x2(host_rows), _ptr(out_row_id),
                      _stream(x_tiled))
    return out, gate_keep, up_keep, hmid


def swiglu_bwd_tiled(gate_keep: torch.Tensor, up_keep: torch.Tensor, elem_offset: int, tiled_rows: int,
                     dh: torch.Tensor, want_hmid: bool = True):
    """(hmid, dgate, dup), row-major like dh [rows, cols], of h = silu(gate) * up for one expert whose gate / up
    projections sit K-tiled in the buffers dual_swiglu_ffn_keep returned, at element offset `elem_offset`, as a
    matrix of `tiled_rows` rows (the expert's row count rounded up to 256).  hmid is None (and not computed) without
    want_hmid: only the down projection's weight gradient reads it."""
    _need_cuda("dh", dh)
    if dh.dtype != torch.bfloat16 or gate_keep.dtype != torch.bfloat16 or up_keep.dtype != torch.bfloat16:
        raise RuntimeError("All tensors must be BFloat16 for this kernel")
    dh = dh.contiguous()
    rows, cols = dh.shape
    hm = torch.empty_like(dh) if want_hmid else None
    dg, du = torch.empty_like(dh), torch.empty_like(dh)
    if rows == 0:
        return hm, dg, du
    with _DeviceGuard(dh):
        _lib.call("wx_swiglu_bwd_tiled", gate_keep.data_ptr() + 2 * elem_offset, up_keep.data_ptr() + 2 * elem_offset,
                  int(tiled_rows), _ptr(dh), _ptr(hm), _ptr(dg), _ptr(du), rows, cols, _stream(dh))
    return hm, dg, du


def dual_swiglu_ffn(x_tiled: torch.Tensor, num_rows: int, expert_offsets: torch.Tensor, weights,
                    hmid: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                    host_rows=None, out_row_id: Optional[torch.Tensor] = None,
                    cache_packed: bool = True, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Both experts' SwiGLU FFN over expert-sorted rows in two launches (act.py:79-82, 142-154).

    x_tiled: result of permute_rows_tiled for num_rows tokens; expert_offsets int32 [3] ON THE DEVICE (from
    partition()); weights = ((gate0, up0, down0), (gate1, up1, down1)) in nn.Linear layout (packed here; the
    packed copies are cached per tensor unless cache_packed is False, or per weight where it is six booleans).  host_rows: optional (rows of expert 0, rows
    of expert 1) as host integers, when the caller has them
    anyway; they only spare the library a second, empty launch when it cannot tell which tile shape fits.
    out_row_id: optional int32 [num_rows] CUDA tensor, the partition's sorted_row_id; with it the result comes back
    in token order (the unpermute happens in the down launch's stores), and `residual` ([num_rows, hidden], token
    order) is added there when given.
    Returns out [num_rows, hidden] bf16, in sorted order unless out_row_id is given.
    """
    (g0, u0, d0), (g1, u1, d1) = weights
    H = g0.size(1)
    I0, I1 = g0.size(0), g1.size(0)
    if tuple(g0.shape) != (I0, H) or tuple(u0.shape) != (I0, H) or tuple(d0.shape) != (H, I0) or \
            tuple(g1.shape) != (I1, H) or tuple(u1.shape) != (I1, H) or tuple(d1.shape) != (H, I1):
        raise RuntimeError("expert weight shapes are inconsistent with hidden size")
    cached = tuple(cache_packed) if isinstance(cache_packed, (tuple, list)) else (bool(cache_packed),) * 6
    packed = [pack_weight(w, cache=c) for w, c in zip((g0, u0, d0, g1, u1, d1), cached)]
    return dual_swiglu_ffn_packed(x_tiled, num_rows, expert_offsets, packed, (H, I0, I1), hmid, out, host_rows,
                                  out_row_id, residual)
