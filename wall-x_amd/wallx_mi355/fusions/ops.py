"""The seven fused ops of wall_x/fusions/ops.py with the same signatures, return values, warnings and
exceptions, running on the MI355X kernels.

    asym_dual_gmm, permute, unpermute, multimodal_rope, get_rope_index, rot_pos_emb, get_window_index
    (ops.py:147, 386, 391, 496, 507, 589, 685)

Differences a caller can observe, all deliberate:
  * multimodal_rope takes a per-call layout= argument.  Its default, "hf", is the channel layout of the model's
    PyTorch path (apply_multimodal_rotary_pos_emb, vl.py:763-769), which is what this build is checked against;
    layout="csrc" gives the layout of the reference's CUDA kernel (csrc/rope.cu:104-117).  The extension-level
    names wallx_csrc.rope / rope_bwd default to "csrc", like the extension they stand in for.
  * bool / int64 expert ids are consumed as they are (no cast kernel); the reference's dtype warning is kept.
  * rot_pos_emb / get_window_index accept grid_thw_host= to skip the device->host read of grid_thw.
"""

import warnings

import torch

from . import backend


# ----------------------------------------------------------------------------- asym_dual_gmm
class AsymmetricDualExpertGemm(torch.autograd.Function):
    """out_e = in_e @ W_e (or W_e^T with trans_b), e in {0, 1}, one launch (ops.py:6-144)."""

    @staticmethod
    def forward(ctx, input_expert0, input_expert1, weight_expert0, weight_expert1, trans_b=False):
        for name, t in (("input_expert0", input_expert0), ("input_expert1", input_expert1),
                        ("weight_expert0", weight_expert0), ("weight_expert1", weight_expert1)):
            assert t.dim() == 2, f"{name} must be 2D"
        k_axis = 1 if trans_b else 0
        assert input_expert0.size(1) == weight_expert0.size(k_axis), \
            f"Expert 0 dimension mismatch (trans_b={trans_b})"
        assert input_expert1.size(1) == weight_expert1.size(k_axis), \
            f"Expert 1 dimension mismatch (trans_b={trans_b})"
        ctx.save_for_backward(input_expert0, input_expert1, weight_expert0, weight_expert1)
        ctx.trans_b = trans_b
        out0, out1 = backend.asym_dual_gmm_separated(input_expert0, input_expert1, weight_expert0,
                                                     weight_expert1, trans_b=trans_b)
        return out0, out1

    @staticmethod
    def backward(ctx, grad_output_expert0, grad_output_expert1):
        in0, in1, w0, w1 = ctx.saved_tensors
        g0, g1 = grad_output_expert0.contiguous(), grad_output_expert1.contiguous()
        # dX = dY @ W^T (weights [k, n]) or dY @ W (weights [n, k])           ops.py:96-107
        gin0, gin1 = backend.asym_dual_gmm_separated(g0, g1, w0, w1, torch.empty_like(in0),
                                                     torch.empty_like(in1), trans_a=False,
                                                     trans_b=not ctx.trans_b)
        # dW = X^T @ dY for [k, n] weights, dY^T @ X for [n, k] weights      ops.py:109-136
        lhs, rhs = ((g0, g1), (in0, in1)) if ctx.trans_b else ((in0, in1), (g0, g1))
        gw0, gw1 = backend.asym_dual_gmm_separated(lhs[0], lhs[1], rhs[0], rhs[1], torch.empty_like(w0),
                                                   torch.empty_like(w1), trans_a=True, trans_b=False)
        return gin0, gin1, gw0, gw1, None


def asym_dual_gmm(input_expert0, input_expert1, weight_expert0, weight_expert1, trans_b=False):
    """(output_expert0 [m0, n0], output_expert1 [m1, n1]); weights [k, n] or [n, k] with trans_b."""
    return AsymmetricDualExpertGemm.apply(input_expert0, input_expert1, weight_expert0, weight_expert1, trans_b)


# ----------------------------------------------------------------------------- permute / unpermute
class PermuteMoE_topK(torch.autograd.Function):
    """ops.py:175-274.  The scratch workspace is cached on the class like the reference's."""

    workspace_fw = None
    dtype = None
    max_expanded_token_num = 0

    @staticmethod
    def forward(ctx, input_act, indices, num_out_tokens, max_token_num):
        if not input_act.numel():
            return input_act, None
        if indices.dim() == 1:
            indices = indices.view(-1, 1)
        if input_act.is_cpu:
            raise RuntimeError("[Error] The input `input_act` of permute_topK op is on the device: CPU!")
        if indices.is_cpu:
            warnings.warn("The input `indices` of permute_topK op is on the device: CPU!")
            indices = indices.to(input_act.device)
        if input_act.size(0) != indices.size(0):
            raise RuntimeError("[Error] permute_topK op input `indices` shape mismatch! "
                               f"Expect {input_act.size(0)}, but got {indices.size(0)}.")
        if indices.dtype != torch.int32:
            warnings.warn(f"The data type of the input `indices` of permute_topK op is {indices.dtype}! "
                          "The recommended type is torch.int32.")
            if indices.dtype not in (torch.int64, torch.bool, torch.uint8):
                indices = indices.to(torch.int32)
        if not input_act.is_contiguous():
            warnings.warn("The input `input_act` of permute_topK op is discontiguous!")
            input_act = input_act.contiguous()
        if not indices.is_contiguous():
            warnings.warn("The input `indices` of permute_topK op is discontiguous!")
            indices = indices.contiguous()

        cls = PermuteMoE_topK
        num_topK = indices.size(1)
        want = max(max_token_num, input_act.size(0)) * num_topK
        if cls.max_expanded_token_num < want:
            cls.max_expanded_token_num = want
            cls.workspace_fw = []
        if cls.dtype != input_act.dtype:
            cls.dtype = input_act.dtype
            cls.workspace_fw = []
        permuted_act, row_id_map, cls.workspace_fw = backend.permute(
            input_act, indices, num_out_tokens, cls.workspace_fw, cls.max_expanded_token_num)
        ctx.row_id_map = row_id_map
        ctx.num_tokens = indices.size(0)
        ctx.num_topK = num_topK
        ctx.mark_non_differentiable(row_id_map)
        return permuted_act, row_id_map

    @staticmethod
    def backward(ctx, permuted_act_grad, _):
        if not permuted_act_grad.numel():
            return permuted_act_grad, None, None, None
        grad = backend.unpermute(permuted_act_grad.contiguous(), ctx.row_id_map, torch.tensor([]),
                                 ctx.num_tokens, ctx.num_topK)
        return grad, None, None, None


class UnpermuteMoE_topK(torch.autograd.Function):
    """ops.py:284-383."""

    @staticmethod
    def forward(ctx, input_act, row_id_map, probs=None):
        if not input_act.numel():
            ctx.probs = probs
            return input_act
        if input_act.is_cpu:
            raise RuntimeError("[Error] The input `input_act` of unpermute_topK op is on the device: CPU!")
        if row_id_map.is_cpu:
            warnings.warn("The input `row_id_map` of unpermute_topK op is on the device: CPU!")
            row_id_map = row_id_map.to(input_act.device)
        if probs is not None and probs.is_cpu:
            warnings.warn("The input `probs` of unpermute_topK op is on the device: CPU!")
            probs = probs.to(input_act.device)
        if probs is not None and row_id_map.size(0) != probs.size(0) * probs.size(1):
            raise RuntimeError("[Error] unpermute_topK op input `probs` shape mismatch! "
                               f"Expect {row_id_map.size(0)}, but got {probs.size(0) * probs.size(1)}.")
        if row_id_map.dtype != torch.int32:
            warnings.warn(f"The data type of the input `row_id_map` of unpermute_topK op is {row_id_map.dtype}! "
                          "The recommended type is torch.int32.")
            row_id_map = row_id_map.to(torch.int32)
        if probs is not None and probs.dtype != torch.float32:
            warnings.warn(f"The data type of the input `probs` of unpermute_topK op is {probs.dtype}! "
                          "The recommended type is torch.float32.")
            probs = probs.to(torch.float32)
        if not input_act.is_contiguous():
            warnings.warn("The input `input_act` of unpermute_topK op is discontiguous!")
            input_act = input_act.contiguous()
        if not row_id_map.is_contiguous():
            warnings.warn("The input `row_id_map` of unpermute_topK op is discontiguous!")
            row_id_map = row_id_map.contiguous()
        if probs is not None and not probs.is_contiguous():
            warnings.warn("The input `probs` of unpermute_topK op is discontiguous!")
            probs = probs.contiguous()

        num_tokens = probs.size(0) if probs is not None else input_act.size(0)
        num_topK = probs.size(1) if probs is not None else 1
        out = backend.unpermute(input_act, row_id_map, probs if probs is not None else torch.tensor([]),
                                num_tokens, num_topK)
        ctx.save_for_backward(input_act, row_id_map, probs)
        return out

    @staticmethod
    def backward(ctx, unpermuted_act_grad):
        if not unpermuted_act_grad.numel():
            return unpermuted_act_grad, None, ctx.probs
        input_act, row_id_map, probs = ctx.saved_tensors
        act_grad = prob_grad = None
        if ctx.needs_input_grad[0]:
            act_grad, prob_grad = backend.unpermute_bwd(unpermuted_act_grad.contiguous(), input_act, row_id_map,
                                                        probs)
        if not ctx.needs_input_grad[2]:
            prob_grad = None
        return act_grad, None, prob_grad


def permute(input_act, indices, num_out_tokens=None, max_token_num=0):
    """(permuted [num_out, H], row_id_map int32 [T*K]); (input_act, None) for an empty input."""
    return PermuteMoE_topK.apply(input_act, indices, 0 if num_out_tokens is None else num_out_tokens,
                                 max_token_num)


def unpermute(input_act, row_id_map, probs=None):
    return UnpermuteMoE_topK.apply(input_act, row_id_map, probs)


# ----------------------------------------------------------------------------- multimodal RoPE
class MultimodalRoPE(torch.autograd.Function):
    """ops.py:402-493.  q [B, Hq, S, D], k [B, Hkv, S, D], cos/sin [3, B, S, D].

    The kernel reads q and k through their strides, so the transposed view of the [B, S, H, D]
    projection output is consumed in place (the reference copies it first, ops.py:437-442).
    Outputs are contiguous [B, H, S, D] like the reference's.
    """

    @staticmethod
    def forward(ctx, q, k, cos, sin, mrope_section, layout="hf"):
        for name, t in (("q", q), ("k", k), ("cos", cos), ("sin", sin)):
            if t.is_cpu:
                raise RuntimeError(f"[Error] The input `{name}` of multimodal_rope op is on the device: CPU!")
        if len(mrope_section) != 3:
            raise RuntimeError("[Error] The input `mrope_section` of multimodal_rope op must be a list of 3 integers!")
        if q.stride(-1) != 1:
            warnings.warn("The input `q` of multimodal_rope op is discontiguous!")
            q = q.contiguous()
        if k.stride(-1) != 1:
            warnings.warn("The input `k` of multimodal_rope op is discontiguous!")
            k = k.contiguous()
        if not cos.is_contiguous():
            warnings.warn("The input `cos` of multimodal_rope op is discontiguous!")
            cos = cos.contiguous()
        if not sin.is_contiguous():
            warnings.warn("The input `sin` of multimodal_rope op is discontiguous!")
            sin = sin.contiguous()
        doubled = [2 * int(v) for v in mrope_section]
        q_out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        k_out = torch.empty(k.shape, dtype=k.dtype, device=k.device)
        backend.rope(q, k, cos, sin, q_out, k_out, doubled, layout)
        ctx.save_for_backward(q, k, cos, sin)
        ctx.mrope_section_doubled = doubled
        ctx.layout = layout
        return q_out, k_out

    @staticmethod
    def backward(ctx, grad_q_out, grad_k_out):
        q, k, cos, sin = ctx.saved_tensors
        want_q, want_k = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        if not (want_q or want_k):
            return None, None, None, None, None, None
        gq = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        gk = torch.empty(k.shape, dtype=k.dtype, device=k.device)
        if grad_q_out.stride(-1) != 1:
            grad_q_out = grad_q_out.contiguous()
        if grad_k_out.stride(-1) != 1:
            grad_k_out = grad_k_out.contiguous()
        backend.rope_bwd(grad_q_out, grad_k_out, q, k, cos, sin, gq, gk, ctx.mrope_section_doubled, ctx.layout)
        return (gq if want_q else None), (gk if want_k else None), None, None, None, None


def multimodal_rope(q, k, cos, sin, mrope_section, layout="hf"):
    """(q', k') = M-RoPE of q and k (ops.py:496-497).  layout="hf": the channel -> plane map of the model's PyTorch
    path (vl.py:763-769); layout="csrc": that of the reference's CUDA kernel (csrc/rope.cu:104-117)."""
    return MultimodalRoPE.apply(q, k, cos, sin, mrope_section, layout)


class MultimodalRoPEFromPositions(torch.autograd.Function):
    """Not in the reference's op set: `multimodal_rope` with Qwen2_5_VLRotaryEmbedding.forward (vl.py:679-712)
    folded in.  Takes position_ids [3, B, S] int64 and inv_freq [D/2] fp32 instead of the cos/sin tables
    [3, B, S, D] built from them, so neither table is ever written or read.  q [B, Hq, S, D], k [B, Hkv, S, D]
    through their strides, contiguous outputs, gradients for q and k only."""

    @staticmethod
    def forward(ctx, q, k, position_ids, inv_freq, mrope_section, layout="hf"):
        for name, t in (("q", q), ("k", k), ("position_ids", position_ids), ("inv_freq", inv_freq)):
            if t.is_cpu:
                raise RuntimeError(f"[Error] The input `{name}` of multimodal_rope op is on the device: CPU!")
        if len(mrope_section) != 3:
            raise RuntimeError("[Error] The input `mrope_section` of multimodal_rope op must be a list of 3 integers!")
        if q.stride(-1) != 1:
            warnings.warn("The input `q` of multimodal_rope op is discontiguous!")
            q = q.contiguous()
        if k.stride(-1) != 1:
            warnings.warn("The input `k` of multimodal_rope op is discontiguous!")
            k = k.contiguous()
        doubled = [2 * int(v) for v in mrope_section]
        inv_freq = inv_freq.to(torch.float32)
        q_out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        k_out = torch.empty(k.shape, dtype=k.dtype, device=k.device)
        backend.rope_from_positions(q, k, position_ids, inv_freq, q_out, k_out, doubled, layout=layout)
        ctx.save_for_backward(position_ids, inv_freq)
        ctx.mrope_section_doubled = doubled
        ctx.layout = layout
        return q_out, k_out

    @staticmethod
    def backward(ctx, grad_q_out, grad_k_out):
        position_ids, inv_freq = ctx.saved_tensors
        want_q, want_k = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        if not (want_q or want_k):
            return None, None, None, None, None, None
        if grad_q_out.stride(-1) != 1:
            grad_q_out = grad_q_out.contiguous()
        if grad_k_out.stride(-1) != 1:
            grad_k_out = grad_k_out.contiguous()
        gq = torch.empty(grad_q_out.shape, dtype=grad_q_out.dtype, device=grad_q_out.device)
        gk = torch.empty(grad_k_out.shape, dtype=grad_k_out.dtype, device=grad_k_out.device)
        backend.rope_from_positions(grad_q_out, grad_k_out, position_ids, inv_freq, gq, gk,
                                    ctx.mrope_section_doubled, backward=True, layout=ctx.layout)
        return (gq if want_q else None), (gk if want_k else None), None, None, None, None


def multimodal_rope_from_positions(q, k, position_ids, inv_freq, mrope_section, layout="hf"):
    return MultimodalRoPEFromPositions.apply(q, k, position_ids, inv_freq, mrope_section, layout)


def multimodal_rope_table(position_ids, inv_freq, mrope_section, layout="hf"):
    """The packed cos/sin table `qkv_projection_with_rope` and `multimodal_rope_from_table` read: build it once per
    forward from the position ids (it replaces the [3, B, S, D] tables of Qwen2_5_VLRotaryEmbedding.forward,
    vl.py:679-712) and hand it to every layer.  layout="hf": the channel -> plane map of the PyTorch path
    (vl.py:763-769; channels d and d + D/2 share an entry, [B*S, D/2]); layout="csrc": that of the reference's CUDA
    kernel (csrc/rope.cu:104-117; one entry per channel, [B*S, D])."""
    if position_ids.is_cpu or inv_freq.is_cpu:
        raise RuntimeError("[Error] The inputs of multimodal_rope_table are on the device: CPU!")
    return backend.mrope_table(position_ids, inv_freq.to(torch.float32), list(mrope_section), layout)


class MultimodalRoPEFromTable(torch.autograd.Function):
    """multimodal_rope with cos / sin read from the packed table of multimodal_rope_table (built once per forward,
    256 or 512 bytes per token, shared by all layers) instead of the two [3, B, S, D] tables; bf16; `layout` as given
    to multimodal_rope_table."""

    @staticmethod
    def forward(ctx, q, k, table, mrope_section, layout="hf"):
        for name, t in (("q", q), ("k", k), ("table", table)):
            if t.is_cpu:
                raise RuntimeError(f"[Error] The input `{name}` of multimodal_rope op is on the device: CPU!")
        if len(mrope_section) != 3:
            raise RuntimeError("[Error] The input `mrope_section` of multimodal_rope op must be a list of 3 integers!")
        if q.stride(-1) != 1:
            warnings.warn("The input `q` of multimodal_rope op is discontiguous!")
            q = q.contiguous()
        if k.stride(-1) != 1:
            warnings.warn("The input `k` of multimodal_rope op is discontiguous!")
            k = k.contiguous()
        doubled = [2 * int(v) for v in mrope_section]
        q_out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        k_out = torch.empty(k.shape, dtype=k.dtype, device=k.device)
        backend.rope_from_table(q, k, table, q_out, k_out, doubled, layout=layout)
        ctx.save_for_backward(table)
        ctx.mrope_section_doubled = doubled
        ctx.layout = layout
        return q_out, k_out

    @staticmethod
    def backward(ctx, grad_q_out, grad_k_out):
        (table,) = ctx.saved_tensors
        want_q, want_k = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        if not (want_q or want_k):
            return None, None, None, None, None
        if grad_q_out.stride(-1) != 1:
            grad_q_out = grad_q_out.contiguous()
        if grad_k_out.stride(-1) != 1:
            grad_k_out = grad_k_out.contiguous()
        gq = torch.empty(grad_q_out.shape, dtype=grad_q_out.dtype, device=grad_q_out.device)
        gk = torch.empty(grad_k_out.shape, dtype=grad_k_out.dtype, device=grad_k_out.device)
        backend.rope_from_table(grad_q_out, grad_k_out, table, gq, gk, ctx.mrope_section_doubled, backward=True,
                                layout=ctx.layout)
        return (gq if want_q else None), (gk if want_k else None), None, None, None


def multimodal_rope_from_table(q, k, table, mrope_section, layout="hf"):
    return MultimodalRoPEFromTable.apply(q, k, table, mrope_section, layout)


class QkvProjectionWithRoPE(torch.autograd.Function):
    """The fused projection under autograd.  Forward: one launch (backend.qkv_rope_proj).  Backward, for the gradient
    `g` of the [B, S, (Hq + 2 Hkv) D] result: the adjoint rotation of g's q and k heads from the same packed table
    (backend.rope_from_table(backward=True), what ops.py:463-493 gives the separate rope op) into a buffer of
    g's shape, the v heads copied beside them; then d hidden = g W and d W = g^T hidden as dual-GEMM launches on the row-major operands (the transposition
    happens inside the kernel) and d bias = the column sums of g (fp32 accumulation, like nn.Linear's)."""

    @staticmethod
    def forward(ctx, hidden_states, qkv_weight, qkv_bias, rope_table, nq, nkv, D, mrope_section, layout):
        out = backend.qkv_rope_proj(hidden_states, qkv_weight, qkv_bias, rope_table, nq, nkv, D)
        ctx.save_for_backward(hidden_states, qkv_weight, rope_table)
        ctx.heads = (nq, nkv, D)
        ctx.rope = ([2 * int(v) for v in mrope_section], layout)
        ctx.has_bias = qkv_bias is not None
        return out

    @staticmethod
    def backward(ctx, grad_out):
        hidden_states, weight, table = ctx.saved_tensors
        nq, nkv, D = ctx.heads
        doubled, layout = ctx.rope
        B, S, H = hidden_states.shape
        N = (nq + 2 * nkv) * D
        go = grad_out.to(torch.bfloat16).contiguous().view(B, S, N)
        g = torch.empty_like(go)  # the gradient w.r.t. the projection's own output: q and k heads rotated back, v as is

        def heads(t, first, count):
            return t[..., first * D:(first + count) * D].view(B, S, count, D).transpose(1, 2)

        backend.rope_from_table(heads(go, 0, nq), heads(go, nq, nkv), table, heads(g, 0, nq), heads(g, nq, nkv), doubled,
                                backward=True, layout=layout)
        g[..., (nq + nkv) * D:].copy_(go[..., (nq + nkv) * D:])
        g2, x2 = g.view(B * S, N), hidden_states.reshape(B * S, H)
        none = g2.new_empty((0, 0))
        want_x, want_w, want_b = ctx.needs_input_grad[0], ctx.needs_input_grad[1], ctx.needs_input_grad[2]
        dx = dw = db = None
        if want_x:  # [T, N] @ [N, H]: the weight is read as stored, K-major
            dx = torch.empty(B * S, H, dtype=torch.bfloat16, device=g.device)
            backend.asym_dual_gmm_separated(g2, none, weight, g2.new_empty((0, H)), dx, g2.new_empty((0, H)), False, False)
            dx = dx.view(B, S, H)
        if want_w:  # [T, N]^T @ [T, H]: both operands K-major
            dw = torch.empty(N, H, dtype=torch.bfloat16, device=g.device)
            backend.asym_dual_gmm_separated(g2, none, x2, g2.new_empty((0, H)), dw, g2.new_empty((0, H)), True, False)
        if want_b and ctx.has_bias:
            db = g2.sum(0, dtype=torch.float32).to(torch.bfloat16)
        return dx, dw, db, None, None, None, None, None, None


def qkv_projection_with_rope(hidden_states, qkv_weight, qkv_bias, rope_table, num_heads, num_key_value_heads,
                             head_dim=128, mrope_section=(16, 24, 24), layout=None):
    """Not in the reference's op set: the first lines of the attention forward (vl.py:955-964) as one launch.

        q = q_proj(h).view(B, S, Hq, D).transpose(1, 2); k, v likewise; q, k = multimodal_rope(q, k, cos, sin, sec)

    hidden_states [B, S, hidden] bf16; qkv_weight / qkv_bias = the q, k and v projections' weights / biases stacked
    along the output dimension (torch.cat((q_proj.weight, k_proj.weight, v_proj.weight)), once per module);
    rope_table from multimodal_rope_table for the same tokens.  Returns (q [B, Hq, S, D], k [B, Hkv, S, D],
    v [B, Hkv, S, D]) as views of one [B, S, (Hq + 2 Hkv) D] buffer (token-major memory, what attention kernels
    take through strides), q and k rotated.  The table's width tells the channel layout it was built for: D / 2
    entries per token reproduce the eager attention class (vl.py:860-862 on the PyTorch rope, vl.py:731-773), D
    entries the flash-attention class, whose rope op runs the CUDA kernel's layout (vl.py:962-964 on
    csrc/rope.cu:104-117).  Differentiable in hidden_states, qkv_weight and qkv_bias; the backward rotates the
    gradient with `mrope_section` / `layout` (the ones the table was built with; layout defaults to the one the
    table's width implies)."""
    if hidden_states.is_cpu:
        raise RuntimeError("[Error] The input `hidden_states` of qkv_projection_with_rope op is on the device: CPU!")
    if hidden_states.dim() != 3:
        raise RuntimeError("[Error] hidden_states must be [batch, seq, hidden]")
    B, S, _ = hidden_states.shape
    D, nq, nkv = head_dim, num_heads, num_key_value_heads
    needs_grad = torch.is_grad_enabled() and (hidden_states.requires_grad or qkv_weight.requires_grad or
                                              (qkv_bias is not None and qkv_bias.requires_grad))
    if needs_grad:
        if len(mrope_section) != 3:
            raise RuntimeError("[Error] The input `mrope_section` of multimodal_rope op must be a list of 3 integers!")
        if layout is None:
            layout = "hf" if rope_table.size(-1) == D // 2 else "csrc"
        out = QkvProjectionWithRoPE.apply(hidden_states, qkv_weight, qkv_bias, rope_table, nq, nkv, D,
                                          tuple(mrope_section), layout)
    else:
        out = backend.qkv_rope_proj(hidden_states, qkv_weight, qkv_bias, rope_table, nq, nkv, D)
    q, k, v = out.split([nq * D, nkv * D, nkv * D], dim=-1)
    return (q.view(B, S, nq, D).transpose(1, 2), k.view(B, S, nkv, D).transpose(1, 2),
            v.view(B, S, nkv, D).transpose(1, 2))


# ----------------------------------------------------------------------------- index builders
def get_rope_index(input_ids, spatial_merge_size, image_token_id, video_token_id, vision_start_token_id,
                   tokens_per_second, image_grid_thw=None, video_grid_thw=None, second_per_grid_ts=None,
                   attention_mask=None):
    """(position_ids int64 [3, B, S], mrope_position_deltas int64 [B, 1]); ops.py:507-579."""
    if not isinstance(input_ids, torch.Tensor):
        raise TypeError("input_ids must be a torch.Tensor")
    if input_ids.dim() != 2:
        raise ValueError("input_ids must be 2D tensor (batch_size, seq_len)")
    if not input_ids.is_cuda:
        raise ValueError("input_ids must be on CUDA device")
    if not isinstance(spatial_merge_size, int) or spatial_merge_size <= 0:
        raise ValueError(f"spatial_merge_size must be positive integer, got {spatial_merge_size}")
    if not isinstance(tokens_per_second, (int, float)) or tokens_per_second <= 0:
        raise ValueError(f"tokens_per_second must be positive number, got {tokens_per_second}")
    return backend.get_rope_index(input_ids, image_grid_thw, video_grid_thw, second_per_grid_ts, attention_mask,
                                  spatial_merge_size, image_token_id, video_token_id, vision_start_token_id,
                                  float(tokens_per_second))


def rot_pos_emb(inv_freq, grid_thw, spatial_merge_size, grid_thw_host=None):
    """fp32 [sum t*h*w, 2*len(inv_freq)] = [h_pos * inv_freq, w_pos * inv_freq]; ops.py:589-675."""
    if not isinstance(inv_freq, torch.Tensor):
        raise TypeError(f"inv_freq must be a torch.Tensor, got {type(inv_freq)}")
    if not isinstance(grid_thw, torch.Tensor):
        raise TypeError(f"grid_thw must be a torch.Tensor, got {type(grid_thw)}")
    if inv_freq.dim() != 1:
        raise ValueError(f"inv_freq must be 1-dimensional, got {inv_freq.dim()}D tensor")
    if grid_thw.dim() != 2:
        raise ValueError(f"grid_thw must be 2-dimensional, got {grid_thw.dim()}D tensor")
    if grid_thw.size(1) != 3:
        raise ValueError(f"grid_thw must have shape [num_grids, 3], got shape {list(grid_thw.shape)}")
    if not inv_freq.is_cuda:
        raise ValueError("inv_freq must be on CUDA device")
    if not grid_thw.is_cuda:
        raise ValueError("grid_thw must be on CUDA device")
    if inv_freq.device != grid_thw.device:
        raise ValueError("inv_freq and grid_thw must be on the same device, "
                         f"got {inv_freq.device} and {grid_thw.device}")
    if not isinstance(spatial_merge_size, int):
        raise TypeError(f"spatial_merge_size must be an integer, got {type(spatial_merge_size)}")
    if spatial_merge_size <= 0:
        raise ValueError(f"spatial_merge_size must be positive, got {spatial_merge_size}")
    if inv_freq.dtype != torch.float32:
        inv_freq = inv_freq.to(torch.float32)
    try:
        return backend.rot_pos_emb(inv_freq, grid_thw, spatial_merge_size, grid_thw_host=grid_thw_host)
    except RuntimeError as e:
        raise RuntimeError(f"CUDA kernel execution failed: {str(e)}")


def get_window_index(grid_thw, window_size, spatial_merge_size, patch_size, spatial_merge_unit=1,
                     grid_thw_host=None):
    """(window_index int32 [N], cu_window_seqlens int32 [W + 1]); ops.py:685-742."""
    assert grid_thw.dim() == 2 and grid_thw.size(1) == 3, \
        f"grid_thw must have shape (num_grids, 3), got {grid_thw.shape}"
    if not grid_thw.is_cuda:
        if grid_thw_host is None:
            grid_thw_host = grid_thw
        grid_thw = grid_thw.cuda()
    if grid_thw.dtype != torch.int32:
        grid_thw = grid_thw.to(torch.int32)
    vit_merger_window_size = window_size // spatial_merge_size // patch_size
    return backend.get_window_index(grid_thw, spatial_merge_size, vit_merger_window_size, patch_size,
                                    spatial_merge_unit, grid_thw_host=grid_thw_host)
