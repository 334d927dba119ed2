"""Prefill harness for BASELINE config 5: a randomly initialised decoder with the Qwen2.5-VL-3B shape and the
dual VL / action expert FFN in every layer (act.py:172-273, 397-530), with every layer's permute, grouped GEMM,
M-RoPE and the position builder replaced by the MI355X kernels.  Attention stays on PyTorch-ROCm
(F.scaled_dot_product_attention), as the configuration prescribes; the QKV / O projections run on this library's
GEMM by default (they carry the rotary embedding and the residual add in their epilogues) or on the vendor's.

This is a measurement harness, not a model port: no KV cache, no generation, no losses; one forward over a
batch of full sequences (prefill).  What it states explicitly:
  * RMSNorm eps 1e-6 (the Qwen2.5-VL-3B value; the reference's config default is 1e-5, cfg.py:179),
  * q/k/v projections with bias, o projection without (vl.py:821-832),
  * attention mask: plain causal by default (`mask="causal"`); `mask="action_block"` adds the reference's
    bidirectional block among action tokens (act.py:616-637): through a dense boolean mask in general, or, when the
    caller states that the action tokens are the last n positions of every row, as two maskless attention calls
    (causal over the prefix; the n action queries over all keys), which is the same function,
  * rotary base 1e6, mrope_section [16, 24, 24], cos/sin built in fp32 and cast to bf16 (vl.py:679-712),
  * `fuse=True` (default) runs the post-attention RMSNorm inside the permute, the residual add AND the next
    reader's RMSNorm (the following layer's input_layernorm, or the final norm) inside the unpermute, M-RoPE
    evaluates cos/sin from the position ids in the kernel (no [3, B, S, D] tables) and leaves q / k token-major,
    and the attention residual is added by the o-projection GEMM; `fuse=False` keeps all of these as separate
    PyTorch ops,
  * `fuse_qkv_rope=True` (default) replaces the vendor GEMM of the q / k / v projection and the rope kernel by one
    launch of this library's GEMM with bias and M-RoPE in its epilogue (vl.py:955-964); `o_proj_native=True`
    (default) runs the o projection with the residual add on this library's row-major GEMM.  With both False the
    projections are vendor GEMMs.
"""

from contextlib import contextmanager
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F

from . import moe, native, workloads as wl
from .fusions import ops


class OpTimer:
    """Accumulates HIP-event durations per op name; events are resolved once, at report time."""

    def __init__(self, enabled: bool = True):
        self.enabled = enabled
        self.pairs: List = []

    @contextmanager
    def section(self, name: str):
        if not self.enabled:
            yield
            return
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        yield
        b.record()
        self.pairs.append((name, a, b))

    def report_ms(self) -> Dict[str, float]:
        torch.cuda.synchronize()
        out: Dict[str, float] = {}
        for name, a, b in self.pairs:
            out[name] = out.get(name, 0.0) + a.elapsed_time(b)
        self.pairs = []
        return out


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return F.rms_norm(x, (x.shape[-1],), weight, eps)


class PrefillHarness:
    def __init__(self, n_layers: int = 36, hidden: int = wl.HIDDEN, n_q: int = wl.N_Q_HEADS, n_kv: int = wl.N_KV_HEADS,
                 head_dim: int = wl.HEAD_DIM, inter=(wl.INTER_VL, wl.INTER_ACT), vocab: int = 151936,
                 eps: float = 1e-6, device="cuda:0", seed: int = 0, mask: str = "causal", keep_dense: bool = False,
                 fuse: bool = True, fuse_qkv_rope: bool = True, o_proj_native: bool = True):
        self.dev = torch.device(device)
        # the q / k / v projection with M-RoPE in its epilogue (one launch of this library's GEMM kernel) instead of
        # the vendor GEMM followed by the rope kernel; needs fuse=True (token-major q / k) and head_dim 128
        self.fuse_qkv_rope = fuse_qkv_rope and fuse and head_dim == 128
        # the o projection with the attention residual added in its epilogue on this library's row-major GEMM
        # (wx_dual_gemm_add, second group empty) instead of the vendor's addmm; needs fuse=True
        self.o_proj_native = o_proj_native and fuse
        self.n_layers, self.hidden, self.n_q, self.n_kv, self.head_dim = n_layers, hidden, n_q, n_kv, head_dim
        self.inter, self.eps, self.mask_mode, self.fuse = inter, eps, mask, fuse
        g = torch.Generator(device=self.dev).manual_seed(seed)

        def w(*shape):
            return (torch.randn(*shape, device=self.dev, generator=g, dtype=torch.float32) * 0.02).to(torch.bfloat16)

        self.embed = w(vocab, hidden)
        self.layers = []
        for _ in range(n_layers):
            layer = {
                "ln1": torch.ones(hidden, dtype=torch.bfloat16, device=self.dev),
                "ln2": torch.ones(hidden, dtype=torch.bfloat16, device=self.dev),
                "wqkv": w((n_q + 2 * n_kv) * head_dim, hidden),  # q, k, v projections in one matrix
                "bqkv": w((n_q + 2 * n_kv) * head_dim),
                "wo": w(hidden, n_q * head_dim),
                "experts": [(w(i, hidden), w(i, hidden), w(hidden, i)) for i in inter],
            }
            # the FFN kernels read K-tiled weights; pack now (static weights) and drop the nn.Linear copies
            layer["packed"] = [tuple(native.pack_weight(t, cache=False) for t in e) for e in layer["experts"]]
            # tests keep the nn.Linear-layout copies (of every layer, or of the listed ones) to evaluate the same
            # weights on the CPU beside this forward
            keep = keep_dense if isinstance(keep_dense, bool) else len(self.layers) in tuple(keep_dense)
            if not keep:
                layer["experts"] = None
            self.layers.append(layer)
        self.final_ln = torch.ones(hidden, dtype=torch.bfloat16, device=self.dev)
        # operands of the empty second group of the o projection's launch
        self._none = (torch.empty(0, n_q * head_dim, dtype=torch.bfloat16, device=self.dev),
                      torch.empty(8, n_q * head_dim, dtype=torch.bfloat16, device=self.dev),
                      torch.empty(0, 8, dtype=torch.bfloat16, device=self.dev))
        self.inv_freq = wl.text_inv_freq(head_dim).to(self.dev)
        self._hmid: Optional[torch.Tensor] = None
        self._x_tiled: Optional[torch.Tensor] = None
        self._ws = None

    # ------------------------------------------------------------------------------------------------
    def _ffn(self, h: torch.Tensor, ln_weight: torch.Tensor, routing: moe.Routing, packed, timer: OpTimer,
             next_norm: Optional[torch.Tensor] = None):
        """h [T, H] (the residual stream after attention) -> (h + FFN(RMSNorm(h)), RMSNorm of that with `next_norm`
        when fused, else None)."""
        from . import _lib

        T, H = h.shape
        I0, I1 = self.inter
        stream = torch.cuda.current_stream().cuda_stream
        rows_pad = native.padded_sorted_rows(T)
        if self._hmid is None or self._hmid.numel() < rows_pad * max(I0, I1):
            self._hmid = torch.empty(rows_pad * max(I0, I1), dtype=torch.bfloat16, device=self.dev)
        if self.fuse:
            with timer.section("rmsnorm+permute"):
                self._x_tiled = native.rmsnorm_permute_rows_tiled(h, ln_weight, self.eps, routing.expert_offsets,
                                                                  routing.sorted_row_id, self._x_tiled)
        else:
            with timer.section("rmsnorm_torch"):
                x = rms_norm(h, ln_weight, self.eps)
            with timer.section("permute"):
                self._x_tiled = native.permute_rows_tiled(x, routing.row_id_map, routing.expert_offsets, self._x_tiled,
                                                          routing.sorted_row_id)
        y_sorted = torch.empty_like(h)
        (g0, u0, d0), (g1, u1, d1) = packed
        with timer.section("ffn_gate_up_swiglu"):
            _lib.call("wx_dual_swiglu_gate_up", self._x_tiled.data_ptr(), self._hmid.data_ptr(),
                      routing.expert_offsets.data_ptr(), g0.data_ptr(), u0.data_ptr(), g1.data_ptr(), u1.data_ptr(),
                      T, H, I0, I1, None, stream)
        with timer.section("ffn_down"):
            _lib.call("wx_dual_down_proj", self._hmid.data_ptr(), y_sorted.data_ptr(), routing.expert_offsets.data_ptr(),
                      d0.data_ptr(), d1.data_ptr(), T, H, I0, I1, None, None, stream)
        if self.fuse:
            with timer.section("unpermute+residual+rmsnorm"):
                return native.unpermute_add_rmsnorm(y_sorted, h, routing.row_id_map, next_norm, self.eps)
        with timer.section("unpermute"):
            y = native.unpermute(y_sorted, routing.row_id_map, torch.tensor([]), T, 1)
        with timer.section("residual_torch"):
            return h + y, None

    @torch.no_grad()
    def forward(self, input_ids: torch.Tensor, image_grid_thw: torch.Tensor, moe_token_types: torch.Tensor,
                timer: Optional[OpTimer] = None, action_suffix: Optional[int] = None,
                capture: Optional[dict] = None) -> torch.Tensor:
        """input_ids [B, S] int64, image_grid_thw [n_img, 3], moe_token_types [B, S] bool -> logits of the last
        position [B, vocab].  action_suffix: with mask="action_block", the caller's statement that the action
        tokens are exactly the last `action_suffix` positions of every row (the data pipeline's layout,
        wall_x/data/utils.py:453-503), which lets the mask be expressed without a dense tensor.
        capture: optional dict with a "layers" entry (layer indices); the forward then leaves in it the position ids
        ("pos") and, per listed layer, what the M-RoPE and FFN kernels read and wrote (q / k before and after the
        rotation, the residual stream before and after the FFN), for checking a full-size forward piece by piece."""
        timer = timer or OpTimer(False)
        B, S = input_ids.shape
        H, D, nq, nkv = self.hidden, self.head_dim, self.n_q, self.n_kv
        with timer.section("rope_index"):
            pos, _ = ops.get_rope_index(input_ids, 2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, 2,
                                        image_grid_thw=image_grid_thw)
        if not self.fuse:
            with timer.section("cos_sin_torch"):
                freqs = pos.float()[..., None] * self.inv_freq
                emb = torch.cat((freqs, freqs), -1)
                cos, sin = emb.cos().to(torch.bfloat16), emb.sin().to(torch.bfloat16)
        with timer.section("partition"):
            ids = moe_token_types.reshape(-1)
            rmap, off, inv, self._ws = native.partition(ids, 2, 0, self._ws, want_sorted=True)
            routing = moe.Routing(rmap, off, ids.numel(), inv)
        if capture is not None:
            capture["pos"] = pos
        rope_table = None
        if self.fuse_qkv_rope:
            with timer.section("mrope_table"):
                rope_table = native.mrope_table(pos, self.inv_freq, wl.MROPE_SECTION)
        attn_mask, n_tail = None, 0
        if self.mask_mode == "action_block":
            if action_suffix is not None:
                # the action tokens are the last `action_suffix` positions of every row: an action query then sees
                # every key of its row (all earlier tokens causally, all action tokens through the block), the other
                # queries stay causal among themselves -- two maskless attention calls instead of a dense mask
                n_tail = int(action_suffix)
            else:
                causal = torch.ones(S, S, dtype=torch.bool, device=self.dev).tril()
                act = moe_token_types[:, None, :, None] & moe_token_types[:, None, None, :]
                attn_mask = causal[None, None] | act
        with timer.section("embed_torch"):
            h = self.embed[input_ids]
        x = None  # RMSNorm of h for the next reader, when the previous layer's closing kernel already made it
        for li, layer in enumerate(self.layers):
            if x is None:
                with timer.section("rmsnorm_torch"):
                    x = rms_norm(h, layer["ln1"], self.eps)
            if self.fuse_qkv_rope:
                with timer.section("qkv_proj+mrope"):
                    qkv = native.qkv_rope_proj(x, layer["wqkv"], layer["bqkv"], rope_table, nq, nkv, D)
                    q, k, v = qkv.split([nq * D, nkv * D, nkv * D], dim=-1)
                    q = q.view(B, S, nq, D).transpose(1, 2)
                    k = k.view(B, S, nkv, D).transpose(1, 2)
                    v = v.view(B, S, nkv, D).transpose(1, 2)
                if capture is not None and li in capture.get("layers", ()):
                    capture[li] = {"x_in": x, "q_out": q, "k_out": k, "v_out": v}
            else:
                with timer.section("qkv_proj_torch"):
                    qkv = F.linear(x, layer["wqkv"], layer["bqkv"])
                    q, k, v = qkv.split([nq * D, nkv * D, nkv * D], dim=-1)
                    q = q.view(B, S, nq, D).transpose(1, 2)
                    k = k.view(B, S, nkv, D).transpose(1, 2)
                    v = v.view(B, S, nkv, D).transpose(1, 2)
                with timer.section("mrope"):
                    if self.fuse:
                        # rotated q / k stay token-major ([B, S, H, D] memory behind the [B, H, S, D] view the kernel
                        # writes through strides), so attention's output comes back token-major as well and the
                        # o projection reads it without a transposing copy
                        qr = torch.empty(B, S, nq, D, dtype=q.dtype, device=self.dev).transpose(1, 2)
                        kr = torch.empty(B, S, nkv, D, dtype=k.dtype, device=self.dev).transpose(1, 2)
                        native.rope_from_positions(q, k, pos, self.inv_freq, qr, kr, [2 * s for s in wl.MROPE_SECTION])
                    else:
                        qr, kr = ops.multimodal_rope(q, k, cos, sin, list(wl.MROPE_SECTION))
                    if capture is not None and li in capture.get("layers", ()):
                        capture[li] = {"q_in": q, "k_in": k, "q_out": qr, "k_out": kr}
                    q, k = qr, kr
            with timer.section("sdpa_torch"):
                if n_tail:
                    head = S - n_tail
                    a = torch.empty_like(q)
                    a[:, :, :head] = F.scaled_dot_product_attention(q[:, :, :head], k[:, :, :head], v[:, :, :head],
                                                                    is_causal=True, enable_gqa=True)
                    a[:, :, head:] = F.scaled_dot_product_attention(q[:, :, head:], k, v, enable_gqa=True)
                else:
                    a = F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask, is_causal=attn_mask is None,
                                                       enable_gqa=True)
            with timer.section("o_proj" if self.o_proj_native else "o_proj_torch"):
                a2d = a.transpose(1, 2).reshape(B * S, nq * D)  # a view when attention kept the token-major layout
                if self.o_proj_native:  # residual in the GEMM's epilogue (rounded product + residual, like eager)
                    res = h.view(B * S, H)
                    h = torch.empty_like(res)
                    native.asym_dual_gmm(a2d, self._none[0], layer["wo"], self._none[1], h, self._none[2], False, True,
                                         add_expert0=res)
                    h = h.view(B, S, H)
                elif self.fuse:
                    h = torch.addmm(h.view(B * S, H), a2d, layer["wo"].t()).view(B, S, H)  # residual in the GEMM
                else:
                    h = h + F.linear(a2d, layer["wo"]).view(B, S, H)
            nxt = self.layers[li + 1]["ln1"] if li + 1 < len(self.layers) else self.final_ln
            ffn_in = h.view(B * S, H)
            h, x = self._ffn(ffn_in, layer["ln2"], routing, layer["packed"], timer, nxt)
            if capture is not None and li in capture.get("layers", ()):
                capture[li].update(ffn_in=ffn_in, ffn_out=h, next_normed=x)
            h = h.view(B, S, H)
            x = x.view(B, S, H) if x is not None else None
        with timer.section("lm_head_torch"):
            last = x[:, -1] if x is not None else rms_norm(h[:, -1], self.final_ln, self.eps)
            logits = F.linear(last, self.embed)
        return logits


def config5_inputs(batch: int = 16, device="cuda:0"):
    """16 sequences x 912 tokens: 768 vision, 112 text-class, 32 action (tail_text = 96 in the config 2 row layout)."""
    ids, grid = wl.config2_tokens(batch=batch, tail_text=96)
    types = ids == wl.ACTION_TOKEN_ID  # load_lerobot_dataset.py:406-409
    return ids.to(device), grid.to(device), types.to(device)
