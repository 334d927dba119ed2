"""Drop-in for the reference's modality-routed MoE block (act.py:67-162) on the fused kernels.

The reference's SparseMoeBlock permutes the tokens, loops over the experts in Python (six cuBLAS GEMMs,
four elementwise kernels and two slice copies per layer, bounds read from CPU tensors) and unpermutes.
Here one layer is: partition (1 or 2 small launches, once per forward: every layer reuses it) -> row gather into
the K-tiled activation layout -> gate/up + SwiGLU for both experts (1 launch) -> down for both experts (1 launch)
whose stores put each row at its token's position (and add the layer's residual when asked to).  Expert weights
are packed into the same K-tiled layout once and cached.  The per-expert row ranges stay on the device
(expert_offsets from the partition), so nothing synchronises with the host.

Parameter names match the reference (``experts.{e}.{gate,up,down}_proj.weight``), so its checkpoints load.
"""

import threading
import weakref
from dataclasses import dataclass
from typing import Optional

import torch
from torch import nn

from . import _lib, native


def activation(name: str):
    """The gating function a config names in `hidden_act` (the reference looks it up in transformers' ACT2FN,
    act.py:73-77): that table when transformers is importable, else the handful of names torch covers."""
    try:
        from transformers.activations import ACT2FN
    except Exception:  # noqa: BLE001 - transformers absent or broken: the local table below
        ACT2FN = None
    if ACT2FN is not None and name in ACT2FN:
        return ACT2FN[name]
    F = torch.nn.functional
    table = {"silu": F.silu, "swish": F.silu, "gelu": F.gelu, "relu": F.relu, "tanh": torch.tanh,
             "sigmoid": torch.sigmoid, "gelu_new": lambda t: F.gelu(t, approximate="tanh"),
             "gelu_pytorch_tanh": lambda t: F.gelu(t, approximate="tanh")}
    if name not in table:
        raise KeyError(f"unknown hidden_act {name!r}")
    return table[name]


class ExpertMLP(nn.Module):
    """Weights of one gated expert, laid out like BlockSparseMLP (act.py:67-82).  The fused kernels implement silu
    gating; an expert with another `hidden_act` makes its block run on the generic ops (see SparseMoeBlock)."""

    def __init__(self, config: dict):
        super().__init__()
        self.hidden_size = config["hidden_size"]
        self.intermediate_size = config["intermediate_size"]
        self.hidden_act = config.get("hidden_act", "silu")
        self.act_fn = activation(self.hidden_act)
        self.gate_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=False)
        self.up_proj = nn.Linear(self.hidden_size, self.intermediate_size, bias=False)
        self.down_proj = nn.Linear(self.intermediate_size, self.hidden_size, bias=False)

    def weights(self):
        return (self.gate_proj.weight, self.up_proj.weight, self.down_proj.weight)


@dataclass
class Routing:
    """Result of the token partition; valid for every layer of a forward pass (token types do not change)."""

    row_id_map: torch.Tensor      # int32 [T]: sorted position of each token
    expert_offsets: torch.Tensor  # int32 [E + 1] on the device
    num_tokens: int
    sorted_row_id: Optional[torch.Tensor] = None  # int32 [T]: token at each sorted position (inverse map)
    host_offsets: Optional[list] = None  # expert_offsets read back to the host (generic path only, once per routing)
    host_rows: Optional["native.HostRows"] = None  # the offsets' asynchronous copy to the host (eager partitions only)

    def rows_when_ready(self):
        """Per-expert row counts as _lib.i64x2 once the partition's asynchronous read-back has landed, else None."""
        return None if self.host_rows is None else self.host_rows.ready()


def _version_of(t: torch.Tensor):
    """The tensor's version counter, or None for a tensor that has none (one created under torch.inference_mode():
    reading `_version` of such a tensor raises).  State derived from a tensor without a counter is never reused:
    nothing would tell a write to it from no write."""
    if t.is_inference():
        return None
    return t._version


class _RoutingCache(threading.local):
    """The partition of the token types last seen on this thread, shared by every block of a model.

    The reference's decoder hands the SAME `moe_token_types` tensor to all of its layers (act.py:257-261, 486), and
    each layer's block would partition it again.  The cache answers with the previous result when the caller passes
    the very same tensor object (so its memory cannot have been recycled for other data), unmodified (same version
    counter), on the same stream and for the same expert count: one partition per forward without any change to
    the reference's model code.  A tensor without a version counter (made under torch.inference_mode()) is partitioned
    on every call.  The partition's scratch buffers are kept here too, per device and stream."""

    def __init__(self):
        self.ref = None
        self.key = None
        self.routing = None
        self.workspace = {}  # (device, stream, capture id) -> [histograms, status word]

    def lookup(self, ids: torch.Tensor, num_experts: int, stream: Optional[int] = None, capture: Optional[int] = None):
        """stream / capture: the current stream's handle and its capture id when the caller has looked them up already
        (a block's forward needs both again for its work buffers)."""
        if stream is None:
            stream = torch.cuda.current_stream(ids.device).cuda_stream if ids.is_cuda else 0
        if capture is None:
            capture = native.capture_id(stream)
        # a partition recorded during a HIP graph capture has not run when the capture ends: it answers lookups of
        # that capture only (its id is part of the key; 0 outside captures)
        version = _version_of(ids)
        key = (version, ids.shape, ids.dtype, ids.device, num_experts, stream, capture)
        if version is not None and self.ref is not None and self.ref() is ids and self.key == key:
            return self.routing
        flat = ids.reshape(-1)
        ws_key = partition_workspace_key(ids.device, stream, key[-1])
        row_id_map, offsets, inverse, ws = native.partition(flat, num_experts, 0, self.workspace.get(ws_key),
                                                            want_sorted=True)
        self.store_workspace(ws_key, ws)
        routing = Routing(row_id_map, offsets, flat.numel(), inverse)
        if key[-1] == 0 and num_experts == 2:  # not under capture: the offsets start their way to the host
            routing.host_rows = native.HostRows(offsets, flat.numel())
        if version is None:  # nothing to check a later call against: answer this call only
            self.ref = self.key = self.routing = None
            return routing
        self.ref, self.key, self.routing = weakref.ref(ids), key, routing
        return routing

    def store_workspace(self, ws_key, ws) -> None:
        """Keeps the partition's scratch pair under its key.  The pair of a capture stays with its graph (a fresh one
        per capture, the pairs of earlier captures are dropped); eager calls keep one per device and stream, so two
        forwards issued on different streams never count into the same histograms."""
        if ws_key[2] != 0:
            for k in [k for k in self.workspace if k[2] not in (0, ws_key[2])]:
                del self.workspace[k]
        if len(self.workspace) >= 64 and ws_key not in self.workspace:
            for k in [k for k in self.workspace if k[2] == 0]:
                del self.workspace[k]
        self.workspace[ws_key] = ws


def partition_workspace_key(device, stream: int, capture: int):
    return (device, stream, capture)


_routing_cache = _RoutingCache()


def _dual(a0, a1, w0, w1, n0, n1, trans_a, trans_b, want=(True, True)):
    """Both experts' products in one launch; an expert whose result nobody asked for (want[e] False) is given an empty
    row range, leaves the launch's tile list, and comes back as None."""
    ref = a0 if a0 is not None else a1

    def absent(n):  # operands of an empty problem with n output columns (either may have been left out by the caller)
        return ref.new_empty((0, 0)), ref.new_empty((n, 0) if trans_b else (0, n))

    if not want[0]:
        a0, w0 = absent(n0)
    if not want[1]:
        a1, w1 = absent(n1)
    m0 = a0.size(1) if trans_a else a0.size(0)
    m1 = a1.size(1) if trans_a else a1.size(0)
    o0 = torch.empty(m0, n0, dtype=torch.bfloat16, device=a0.device)
    o1 = torch.empty(m1, n1, dtype=torch.bfloat16, device=a0.device)
    native.asym_dual_gmm(a0, a1, w0, w1, o0, o1, trans_a, trans_b)
    return (o0 if want[0] else None), (o1 if want[1] else None)


_cu_counts = {}


def _cus(device: torch.device) -> int:
    n = _cu_counts.get(device.index)
    if n is None:
        n = _cu_counts[device.index] = torch.cuda.get_device_properties(device).multi_processor_count
    return n


def _weight_grads(a0, a1, b0, b1, n0, n1, want):
    """The experts' weight gradients dW_e = a_e^T b_e (a_e [rows_e, out_e], b_e [rows_e, n_e]: the contraction runs over
    the expert's tokens) as one launch, like _dual -- unless the wide expert's output is an awkward number of 256 x 256
    tiles for the chip.  11008 x 2048 is 344 tiles: two rounds on 256 CUs for 1.34 rounds of work.  Its contraction
    is tens of thousands of tokens long, so it is cut in two: both halves go into one launch as its two problems (688
    tiles of half the length: three rounds of half the time), their bf16 results are added, and the narrow expert's
    gradient (a few cheap tiles) takes a launch of its own.  The sum of two rounded halves carries one rounding more
    than the single product; the gradient tests' tolerance covers it."""
    if want[0] and a0.size(0) >= 4096:
        cus = _cus(a0.device)
        tiles = -(-a0.size(1) // 256) * -(-n0 // 256)
        if -(-2 * tiles // cus) < 2 * -(-tiles // cus):
            h = a0.size(0) // 2
            first, second = _dual(a0[:h], a0[h:], b0[:h], b0[h:], n0, n0, True, False)
            first.add_(second)
            other = _dual(None, a1, None, b1, n0, n1, True, False, want=(False, True))[1] if want[1] else None
            return first, other
    return _dual(a0, a1, b0, b1, n0, n1, True, False, want=want)


class _MoeBlockFunction(torch.autograd.Function):
    """[RMSNorm ->] permute -> both experts' SwiGLU FFN -> unpermute [+ residual] with a backward (act.py:105-162,
    and the decoder layer's lines around it, act.py:256-265, under autograd).

    Forward is the fused path; its gate / up launch also keeps the two projections (the reference's autograd keeps
    them too, along with act_fn(gate) and the product, act.py:79-82).  With a norm weight the post-attention RMSNorm
    runs inside the permute, with `residual` the closing add inside the down launch's stores.  Backward runs every
    remaining contraction of both experts as one dual GEMM each: dHm = dY Wd, dWd = dY^T Hm, dX = dG Wg + dU Wu (the
    second product added onto the first in its epilogue), dWg = dG^T X, dWu = dU^T X,
    with the SwiGLU derivative (and Hm in row-major form) from one fused elementwise kernel per expert (fp32 math).
    The normed, sorted rows the weight gradients contract over are recomputed (one pass, where the plain block
    permutes x), and the unpermute of dX carries the norm's backward and the residual branch's gradient (one pass,
    which also sums the norm weight's gradient).  Intermediate sizes that are not multiples of 64 recompute the two
    projections instead.  The per-expert row counts come from the partition's asynchronous read-back (Routing.host_rows);
    only a routing without one makes the backward wait for a copy of expert_offsets (the forward never synchronises)."""

    N_FIXED = 8  # inputs in front of the six weights

    @staticmethod
    def forward(ctx, x, norm_weight, row_id_map, expert_offsets, sorted_row_id, scratch, eps, residual, *weights):
        T = x.size(0)
        if norm_weight is not None:
            if sorted_row_id is None:
                raise RuntimeError("pre_norm needs a routing with sorted_row_id (partition(..., want_sorted=True))")
            scratch["x_tiled"] = native.rmsnorm_permute_rows_tiled(x, norm_weight, eps, expert_offsets, sorted_row_id,
                                                                   scratch.get("x_tiled"))
        else:
            scratch["x_tiled"] = native.permute_rows_tiled(x, row_id_map, expert_offsets, scratch.get("x_tiled"),
                                                           sorted_row_id)
        w = ((weights[0], weights[1], weights[2]), (weights[3], weights[4], weights[5]))
        I0, I1 = weights[0].size(0), weights[3].size(0)
        ctx.keep = I0 % 64 == 0 and I1 % 64 == 0
        ctx.eps, ctx.residual, ctx.has_norm = eps, bool(residual), norm_weight is not None
        ctx.has_sorted = sorted_row_id is not None
        # weights that train are repacked on every forward: writes through `.data` (master-weight or EMA copies) do
        # not move the version counter a cached copy would be checked against.  Frozen ones keep their packed copies.
        n0 = _MoeBlockFunction.N_FIXED
        frozen = tuple(not n for n in ctx.needs_input_grad[n0:n0 + 6])
        res_in_stores = x if (residual and sorted_row_id is not None) else None
        # the partition's own read-back of the row counts, once it has landed (never consulted while capturing): one
        # dispatch per GEMM in the forward, and a backward that starts without a synchronisation
        ctx.rows_when_ready = scratch.get("rows_when_ready")
        rows = None
        if ctx.rows_when_ready is not None and \
                native.capture_id(torch.cuda.current_stream(x.device).cuda_stream) == 0:
            rows = ctx.rows_when_ready()
        saved = [x, row_id_map, expert_offsets]
        if ctx.has_norm:
            saved.append(norm_weight)
        if ctx.has_sorted:
            saved.append(sorted_row_id)
        if ctx.keep:
            y, gate_keep, up_keep, scratch["hmid"] = native.dual_swiglu_ffn_keep(
                scratch["x_tiled"], T, expert_offsets, w, hmid=scratch.get("hmid"), host_rows=rows,
                out_row_id=sorted_row_id, frozen=frozen, residual=res_in_stores)
            saved += [gate_keep, up_keep]
        else:
            y = native.dual_swiglu_ffn(scratch["x_tiled"], T, expert_offsets, w, hmid=scratch.get("hmid"),
                                       host_rows=rows, out_row_id=sorted_row_id, cache_packed=frozen,
                                       residual=res_in_stores)
        ctx.save_for_backward(*saved, *weights)
        if sorted_row_id is None:
            if residual:
                return native.unpermute_add(y, x, row_id_map)
            return native.unpermute(y, row_id_map, torch.tensor([]), T, 1)
        return y

    @staticmethod
    def backward(ctx, dy):
        saved = list(ctx.saved_tensors)
        x, row_id_map, expert_offsets = saved[:3]
        del saved[:3]
        norm_weight = saved.pop(0) if ctx.has_norm else None
        sorted_row_id = saved.pop(0) if ctx.has_sorted else None
        gate_keep, up_keep = (saved.pop(0), saved.pop(0)) if ctx.keep else (None, None)
        g0, u0, d0, g1, u1, d1 = saved
        T, H = x.shape
        n0 = _MoeBlockFunction.N_FIXED
        need = (None,) * 5 + tuple(ctx.needs_input_grad[n0:n0 + 6])  # need[5..10]: the six weights
        need_x, need_norm = ctx.needs_input_grad[0], ctx.has_norm and ctx.needs_input_grad[1]
        rows = ctx.rows_when_ready() if ctx.rows_when_ready is not None else None
        if rows is not None:
            m0, m1 = int(rows[0]), int(rows[1])
        else:  # no read-back under way (a routing made by hand or under capture), or it has not landed: wait for one
            o = expert_offsets.cpu().tolist()
            m0, m1 = o[1] - o[0], o[2] - o[1]
        dy = dy.contiguous().to(torch.bfloat16)
        if ctx.has_norm:  # the experts' input rows: normed, in sorted order
            xs = native.rmsnorm_permute_rows(x.detach(), norm_weight.detach(), ctx.eps, sorted_row_id)
        else:
            xs = native.permute_rows(x.detach(), row_id_map, 1, T)
        dys = native.permute_rows(dy, row_id_map, 1, T)
        x0, x1 = xs[:m0], xs[m0:m0 + m1]
        dy0, dy1 = dys[:m0], dys[m0:m0 + m1]
        I0, I1 = g0.size(0), g1.size(0)
        dh0, dh1 = _dual(dy0, dy1, d0, d1, I0, I1, False, False)
        if ctx.keep:
            pad0 = (m0 + 255) // 256 * 256
            pad1 = (m1 + 255) // 256 * 256
            # the forward's hmid in row-major form is read by the down projection's weight gradient only
            hm0, dg0, du0 = native.swiglu_bwd_tiled(gate_keep, up_keep, 0, pad0, dh0, want_hmid=need[7])
            hm1, dg1, du1 = native.swiglu_bwd_tiled(gate_keep, up_keep, pad0 * I0, pad1, dh1, want_hmid=need[10])
        else:
            ga0, ga1 = _dual(x0, x1, g0, g1, I0, I1, False, True)
            up0, up1 = _dual(x0, x1, u0, u1, I0, I1, False, True)
            hm0, dg0, du0 = native.swiglu_bwd(ga0, up0, dh0)
            hm1, dg1, du1 = native.swiglu_bwd(ga1, up1, dh1)
        grads = [None] * 6
        # weight gradients only of the experts that train: fine-tuning with the VL side frozen (the reference's
        # freeze_vlm mode trains `moe.experts.1.*` alone, qwen_vl_act_trainer.py:530-536) skips the three large ones
        if need[5] or need[8]:  # gate weights
            grads[0], grads[3] = _weight_grads(dg0, dg1, x0, x1, H, H, (need[5], need[8]))
        if need[6] or need[9]:  # up weights
            grads[1], grads[4] = _weight_grads(du0, du1, x0, x1, H, H, (need[6], need[9]))
        if need[7] or need[10]:  # down weights
            grads[2], grads[5] = _weight_grads(dy0, dy1, hm0, hm1, I0, I1, (need[7], need[10]))
        dx = dnorm = None
        if need_x or need_norm:
            # dX = dG Wg + dU Wu: the second product accumulates onto the first in its epilogue (bf16 + bf16, rounded
            # once -- what the two eager ops and their add give)
            dxs = torch.empty(T, H, dtype=torch.bfloat16, device=x.device)
            d0_, d1_ = dxs[:m0], dxs[m0:m0 + m1]
            native.asym_dual_gmm(dg0, dg1, g0, g1, d0_, d1_, False, False)
            native.asym_dual_gmm(du0, du1, u0, u1, d0_, d1_, False, False, add_expert0=d0_, add_expert1=d1_)
            if ctx.has_norm:
                dx, dnorm = native.unpermute_rmsnorm_bwd(dxs, x.detach(), norm_weight.detach(), ctx.eps, row_id_map,
                                                         add=dy if ctx.residual else None)
            elif ctx.residual:
                dx = native.unpermute_add(dxs, dy, row_id_map)
            else:
                dx = native.unpermute(dxs, row_id_map, torch.tensor([]), T, 1)
        elif ctx.residual and need_x:
            dx = dy
        return (dx if need_x else None, dnorm if need_norm else None, None, None, None, None, None, None, *grads)


class SparseMoeBlock(nn.Module):
    """Same constructor and forward signature as the reference block (act.py:85-162).

    wall-x's own configuration -- two silu-gated experts of one hidden size -- runs the fused dual-expert path.  Any
    other `config.experts` list (another expert count, another `hidden_act`) runs the same block on this library's
    generic ops instead: `ops.permute`, then per pair of experts `ops.asym_dual_gmm` for the gate, up and down
    projections with the activation as a torch op between them, then `ops.unpermute` (all differentiable)."""

    def __init__(self, config, num_experts: int):
        super().__init__()
        self.num_experts = num_experts
        self.experts = nn.ModuleList([ExpertMLP(config.experts[i]) for i in range(num_experts)])
        self._fused = (num_experts == 2 and all(e.hidden_act in ("silu", "swish") for e in self.experts) and
                       self.experts[0].hidden_size == self.experts[1].hidden_size)
        self._dims = (self.experts[0].hidden_size, self.experts[0].intermediate_size,
                      self.experts[1].intermediate_size) if self._fused else None
        self._hmid: Optional[torch.Tensor] = None      # training path only; inference shares buffers per stream
        self._x_tiled: Optional[torch.Tensor] = None
        self._packed: Optional[native.PackedExperts] = None  # set by pack_for_inference()
        self._rows_seen = None

    def route(self, experts_indices: torch.Tensor) -> Routing:
        """Stable partition of the flattened token types.  The result is valid for all layers of a forward; it is
        remembered (per thread) for as long as the caller keeps passing the same, unmodified tensor object, which is
        what the reference's decoder does for its 36 layers (act.py:257-261)."""
        return _routing_cache.lookup(experts_indices, self.num_experts)

    def pack_for_inference(self, free_dense: bool = True) -> "SparseMoeBlock":
        """Packs the six projection weights into the K-tiled layout the kernels read and, with free_dense, releases
        the nn.Linear copies (the parameters stay registered, emptied, so the module tree keeps its shape): half the
        expert memory of a block that holds both.  The block is forward-only afterwards; load weights first."""
        if not self._fused:
            raise RuntimeError("pack_for_inference: only the fused dual-expert configuration (two silu experts) has a "
                               "packed form; this block runs on the generic ops")
        flat = [w for e in self.experts for w in e.weights()]
        if any(w.numel() == 0 for w in flat):
            raise RuntimeError("pack_for_inference: the nn.Linear weights were already released")
        self._packed = native.PackedExperts([native.pack_weight(w.detach(), cache=False) for w in flat], self._dims)
        if free_dense:
            for e in self.experts:
                for proj in (e.gate_proj, e.up_proj, e.down_proj):
                    native.invalidate_packed(proj.weight)
                    proj.weight = nn.Parameter(torch.empty(0, dtype=proj.weight.dtype, device=proj.weight.device),
                                               requires_grad=False)
        return self

    def forward(self, hidden_states: torch.Tensor, experts_indices: torch.Tensor,
                start_indices: Optional[torch.Tensor] = None, end_indices: Optional[torch.Tensor] = None,
                routing: Optional[Routing] = None, pre_norm=None, residual: bool = False) -> torch.Tensor:
        """hidden_states [B, S, H] bf16; experts_indices [B, S] (bool or integer expert id).

        start_indices / end_indices (the reference's CPU tensors of per-expert row ranges, act.py:1274-1283) are
        optional: the kernels take the row ranges from the partition on the device; when the caller passes them
        anyway, their lengths tell the library which tile shape fits without a second launch.

        Two optional caller fusions (the decoder layer around this block, act.py:256-265):
        pre_norm=(weight, eps) applies the post-attention RMSNorm to hidden_states inside the permute, and
        residual=True returns hidden_states + block(...) with the add done in the down launch's stores.  With both, the
        layer's `residual = h; h = norm(h); h = moe(h); h = residual + h` is `h = moe(h, ..., pre_norm, True)`.
        """
        batch, seq, hidden = hidden_states.shape
        x = hidden_states.reshape(-1, hidden)
        if x.dtype != torch.bfloat16:
            # under bf16 autocast (the reference trains with accelerate's mixed_precision="bf16", train_qact.py:65) the
            # nn.Linear layers this block replaces would take an fp32 input and answer in bf16: do the same
            if x.is_floating_point() and torch.is_autocast_enabled("cuda") and \
                    torch.get_autocast_dtype("cuda") == torch.bfloat16:
                x = x.to(torch.bfloat16)
            else:
                raise RuntimeError("All tensors must be BFloat16 for this kernel")
        T = x.size(0)
        if not self._fused:
            return self._forward_generic(x, experts_indices, start_indices, end_indices, routing, pre_norm,
                                         residual).view(batch, seq, hidden)
        host_rows = self._host_rows(start_indices, end_indices, T)
        # the stream and its capture state, looked up once for the partition cache and the work buffers
        stream = torch.cuda.current_stream(x.device).cuda_stream if x.is_cuda else 0
        capture = native.capture_id(stream) if x.is_cuda else 0
        if routing is None:
            routing = _routing_cache.lookup(experts_indices, self.num_experts, stream, capture)
        if routing.num_tokens != T:
            raise RuntimeError(f"routing was built for {routing.num_tokens} tokens, got {T}")
        grad = torch.is_grad_enabled()
        if self._packed is not None:
            if grad and x.requires_grad:
                raise RuntimeError("a block packed for inference has no backward")
            experts = self._packed
        else:
            flat = [w for e in self.experts for w in e.weights()]
            if grad and (x.requires_grad or any(w.requires_grad for w in flat)):
                return self._forward_training(x, routing, flat, pre_norm, residual).view(batch, seq, hidden)
            # frozen nn.Linear weights: packed once, the copies checked against storage and version on every call
            experts = _experts_for((flat[:3], flat[3:]))
        if routing.sorted_row_id is None:
            return self._forward_scatter(x, routing, experts, host_rows, pre_norm, residual).view(batch, seq, hidden)
        return native.packed_block_forward(experts, x, routing.row_id_map, routing.sorted_row_id,
                                           routing.expert_offsets, host_rows, pre_norm, residual,
                                           routing.rows_when_ready, stream, capture).view(batch, seq, hidden)

    def _host_rows(self, start_indices, end_indices, num_tokens):
        """The per-expert row counts as a host int64[2] when the caller's CPU tensors give them, else None.  The
        answer is kept for as long as the caller passes the same two unmodified tensor objects (the reference
        builds them once per forward, act.py:1274-1283, and hands them to all 36 layers)."""
        if start_indices is None or end_indices is None or start_indices.is_cuda or end_indices.is_cuda:
            return None
        versions = (_version_of(start_indices), _version_of(end_indices))
        tracked = None not in versions  # tensors made under inference_mode have no counter: read them every call
        hit = self._rows_seen
        if tracked and hit is not None and hit[0] is start_indices and hit[1] is end_indices and \
                hit[2] == (*versions, num_tokens):
            return hit[3]
        counts = (end_indices - start_indices).tolist()
        rows = None
        if len(counts) == 2 and min(counts) >= 0 and sum(counts) == num_tokens:
            rows = _lib.i64x2(counts)
        self._rows_seen = (start_indices, end_indices, (*versions, num_tokens), rows) if tracked else None
        return rows

    def _forward_training(self, x, routing, flat, pre_norm, residual):
        # the norm runs inside the permute and the residual add inside the down launch's stores, as in the inference
        # path; the autograd function's backward covers both
        norm_weight, eps = pre_norm if pre_norm is not None else (None, 0.0)
        need = native.padded_sorted_rows(x.size(0)) * max(self._dims[1:])
        if self._hmid is None or self._hmid.numel() < need or self._hmid.device != x.device:
            self._hmid = torch.empty(need, dtype=torch.bfloat16, device=x.device)
        scratch = {"x_tiled": self._x_tiled, "hmid": self._hmid, "rows_when_ready": routing.rows_when_ready}
        y = _MoeBlockFunction.apply(x, norm_weight, routing.row_id_map, routing.expert_offsets,
                                    routing.sorted_row_id, scratch, float(eps), bool(residual), *flat)
        self._x_tiled = scratch["x_tiled"]
        return y

    def _forward_generic(self, x, experts_indices, start_indices, end_indices, routing, pre_norm, residual):
        """Any expert list (act.py:105-162 as written): permute -> per pair of experts the three projections as
        dual GEMMs with the activation between them -> unpermute.  Row ranges come from the caller's CPU tensors when
        given (act.py:1274-1283), else from the partition's offsets, read back once per routing."""
        from .fusions import ops

        E, T = self.num_experts, x.size(0)
        xin = x
        if pre_norm is not None:
            norm_weight, eps = pre_norm
            xin = torch.nn.functional.rms_norm(x, (x.size(1),), norm_weight, eps)
        bounds = None
        if start_indices is not None and end_indices is not None and not start_indices.is_cuda \
                and not end_indices.is_cuda:
            starts, ends = start_indices.tolist(), end_indices.tolist()
            if len(starts) == E and len(ends) == E:
                bounds = list(zip((int(v) for v in starts), (int(v) for v in ends)))
        if bounds is None:
            if routing is None:
                routing = _routing_cache.lookup(experts_indices, E)
            if routing.host_offsets is None:
                routing.host_offsets = routing.expert_offsets.cpu().tolist()
            off = routing.host_offsets
            bounds = [(off[e], off[e + 1]) for e in range(E)]
        if T == 0:
            return xin + x if residual else xin
        ids = experts_indices.reshape(-1)
        permuted, row_id_map = ops.permute(xin, ids if ids.dtype == torch.int32 else ids.to(torch.int32))
        final = torch.zeros_like(permuted)  # rows no expert range covers stay zero (act.py:139)
        for e in range(0, E, 2):
            a, b = self.experts[e], self.experts[e + 1] if e + 1 < E else None
            ra, rb = bounds[e], bounds[e + 1] if b is not None else (0, 0)
            if ra[0] == ra[1] and rb[0] == rb[1]:
                continue  # act.py:144-145
            xa = permuted[ra[0]:ra[1]]
            if b is not None:
                xb, wb, act_b = permuted[rb[0]:rb[1]], b.weights(), b.act_fn
            else:  # an odd expert count: the last launch's second problem is empty
                xb = permuted.new_empty((0, a.hidden_size))
                wb = (permuted.new_empty((8, a.hidden_size)), permuted.new_empty((8, a.hidden_size)),
                      permuted.new_empty((a.hidden_size, 8)))
                act_b = a.act_fn
            wa = a.weights()
            ga, gb = ops.asym_dual_gmm(xa, xb, wa[0], wb[0], trans_b=True)
            ua, ub = ops.asym_dual_gmm(xa, xb, wa[1], wb[1], trans_b=True)
            ya, yb = ops.asym_dual_gmm(a.act_fn(ga) * ua, act_b(gb) * ub, wa[2], wb[2], trans_b=True)
            if ra[0] != ra[1]:
                final[ra[0]:ra[1]] = ya
            if rb[0] != rb[1]:
                final[rb[0]:rb[1]] = yb
        y = ops.unpermute(final, row_id_map)
        return x + y if residual else y

    def _forward_scatter(self, x, routing, experts, host_rows, pre_norm, residual):
        # a caller's Routing without the inverse map: scatter rows by row_id_map, separate unpermute
        if pre_norm is not None:
            raise RuntimeError("pre_norm needs a routing with sorted_row_id (partition(..., want_sorted=True))")
        x_tiled = native.permute_rows_tiled(x, routing.row_id_map, routing.expert_offsets, None, None)
        y_sorted = native.dual_swiglu_ffn_packed(x_tiled, x.size(0), routing.expert_offsets, experts.tensors,
                                                 self._dims, host_rows=host_rows)
        if residual:
            return native.unpermute_add(y_sorted, x, routing.row_id_map)
        return native.unpermute(y_sorted, routing.row_id_map, torch.tensor([]), x.size(0), 1)


_functional_experts = {}  # ids of the six weight tensors -> (their storage / version state, weak references, PackedExperts)


native._invalidate_hooks.append(lambda _w: _functional_experts.clear())


def _experts_for(weights) -> "native.PackedExperts":
    """PackedExperts for weights given as ((gate0, up0, down0), (gate1, up1, down1)) in nn.Linear layout: packed
    once per set of tensors and reused while those tensor objects keep their storage and version counters."""
    flat = (*weights[0], *weights[1])
    key = tuple(map(id, flat))
    state = tuple((w.data_ptr(), _version_of(w)) for w in flat)
    tracked = all(v is not None for _, v in state)  # weights made under inference_mode: packed on every call
    hit = _functional_experts.get(key) if tracked else None
    if hit is not None and hit[0] == state and all(r() is w for r, w in zip(hit[1], flat)):
        return hit[2]
    g0, u0, d0, g1, u1, d1 = flat
    H, I0, I1 = g0.size(1), g0.size(0), g1.size(0)
    if tuple(u0.shape) != (I0, H) or tuple(d0.shape) != (H, I0) or tuple(g1.shape) != (I1, H) or \
            tuple(u1.shape) != (I1, H) or tuple(d1.shape) != (H, I1):
        raise RuntimeError("expert weight shapes are inconsistent with hidden size")
    experts = native.PackedExperts([native.pack_weight(w, cache=tracked) for w in flat], (H, I0, I1))
    if not tracked:
        return experts
    if len(_functional_experts) >= 64:
        _functional_experts.clear()
    # the entry (and with it the packed copies) goes when any of the six tensors does
    refs = [weakref.ref(w, lambda _r, k=key: _functional_experts.pop(k, None)) for w in flat]
    _functional_experts[key] = (state, refs, experts)
    return experts


def moe_layer_forward(x: torch.Tensor, token_types: torch.Tensor, weights, routing: Optional[Routing] = None,
                      hmid: Optional[torch.Tensor] = None, workspace=None, host_rows=None):
    """Functional form of one layer: permute -> dual-expert SwiGLU FFN -> unpermute.

    x [T, H] bf16, token_types [T] (bool / int), weights ((g0,u0,d0),(g1,u1,d1)).  Returns (y [T, H], routing).
    Without `routing` the token types are partitioned on every call (pass the returned routing to the following
    layers; a caller that knows the per-expert row counts passes `host_rows` too -- unlike the block's cached
    partition, this one starts no read-back of its own, which would cost a call that is not repeated more than it
    saves).  Frozen weights are packed once (see native.pack_weight for what invalidates the packed copies); the
    work buffers are the per-stream pair every block shares, so `hmid` is accepted for compatibility and not used.
    """
    if routing is None:
        stream = torch.cuda.current_stream(token_types.device).cuda_stream
        ws_key = partition_workspace_key(token_types.device, stream, native.capture_id(stream))
        ws = workspace if workspace is not None else _routing_cache.workspace.get(ws_key)
        row_id_map, offsets, inverse, ws = native.partition(token_types.reshape(-1), 2, 0, ws, want_sorted=True)
        if workspace is None:
            _routing_cache.store_workspace(ws_key, ws)
        routing = Routing(row_id_map, offsets, x.size(0), inverse)
    experts = _experts_for(weights)
    rows = None if host_rows is None else _lib.i64x2(host_rows)
    if routing.sorted_row_id is not None:  # the down launch stores every row at its token's position
        y = native.packed_block_forward(experts, x, routing.row_id_map, routing.sorted_row_id,
                                        routing.expert_offsets, rows, rows_when_ready=routing.rows_when_ready)
        return y, routing
    x_tiled = native.permute_rows_tiled(x, routing.row_id_map, routing.expert_offsets, None, None)
    y_sorted = native.dual_swiglu_ffn_packed(x_tiled, x.size(0), routing.expert_offsets, experts.tensors,
                                             (experts.hidden, experts.inter0, experts.inter1), host_rows=host_rows)
    y = native.unpermute(y_sorted, routing.row_id_map, torch.tensor([]), x.size(0), 1)
    return y, routing
