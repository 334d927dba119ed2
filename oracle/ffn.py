"""Oracle: dual-expert grouped GEMM and SwiGLU FFN (test infrastructure only).

Follows ops.py:6-165 / csrc/dual_asym_grouped_gemm.cu:308-366 for the grouped
GEMM contract and act.py:67-162 for the expert FFN and the MoE block.
"""

import torch
import torch.nn.functional as F


def dual_gemm_ref(in0, in1, w0, w1, trans_a: bool = False, trans_b: bool = False,
                  out_dtype=None):
    """out_e = op(in_e) @ op(w_e), e in {0, 1}; fp32 accumulation, one rounding.

    csrc/dual_asym_grouped_gemm.cu:49-136: bf16 operands, fp32 accumulator,
    epilogue alpha = 1, beta = 0 (:257).  ``trans_b`` means the weight is stored
    [n, k] (the nn.Linear layout); ``trans_a`` means the input is stored [k, m].
    """
    outs = []
    for a, w in ((in0, w0), (in1, w1)):
        a32 = a.to(torch.float32)
        w32 = w.to(torch.float32)
        if trans_a:
            a32 = a32.t()
        if trans_b:
            w32 = w32.t()
        o = a32 @ w32
        outs.append(o.to(out_dtype or a.dtype))
    return outs[0], outs[1]


def activation_ref(name: str):
    """The gating function named by an expert's `hidden_act` (act.py:73,77 looks the name up in transformers'
    ACT2FN): written out here for the names a wall-x style config can carry."""
    table = {
        "silu": F.silu,
        "swish": F.silu,
        "gelu": F.gelu,  # the exact (erf) form
        "gelu_new": lambda t: F.gelu(t, approximate="tanh"),
        "gelu_pytorch_tanh": lambda t: F.gelu(t, approximate="tanh"),
        "relu": F.relu,
    }
    return table[name]


def swiglu_ffn_ref(x, gate_w, up_w, down_w, eager_rounding: bool = True, act: str = "silu"):
    """down(act(gate(x)) * up(x)) with nn.Linear weights [out, in] (act.py:74-82); act = the expert's
    `hidden_act`, silu in wall-x's own configuration.

    eager_rounding=True reproduces the reference's op-by-op evaluation in the
    activation dtype: every F.linear / silu / multiply result is rounded to
    x.dtype before the next op (what nn.Linear + ACT2FN["silu"] do in bf16), with
    fp32 accumulation inside each matmul.  eager_rounding=False keeps fp32
    throughout and rounds once at the end.
    """
    dt = x.dtype
    fn = activation_ref(act)
    x32 = x.to(torch.float32)
    g = x32 @ gate_w.to(torch.float32).t()
    u = x32 @ up_w.to(torch.float32).t()
    if eager_rounding:
        g = g.to(dt).to(torch.float32)
        u = u.to(dt).to(torch.float32)
        a = fn(g).to(dt).to(torch.float32)
        h = (a * u).to(dt).to(torch.float32)
    else:
        h = fn(g) * u
    y = h @ down_w.to(torch.float32).t()
    return y.to(dt)


def swiglu_bwd_ref(gate, up, dh):
    """(hmid, dgate, dup) for h = silu(gate) * up (act.py:79-82) and the gradient dh w.r.t. h.

    The reference leaves this to autograd; so does this restatement (torch.autograd on the fp32 expression), with
    hmid carrying the forward's eager rounding (silu rounded to the activation dtype before the product) and each
    result rounded once.
    """
    dt = gate.dtype
    g = gate.to(torch.float32).clone().requires_grad_(True)
    u = up.to(torch.float32).clone().requires_grad_(True)
    h = F.silu(g) * u
    dg, du = torch.autograd.grad(h, (g, u), dh.to(torch.float32))
    hm = (F.silu(g.detach()).to(dt).to(torch.float32) * u.detach()).to(dt)
    return hm, dg.to(dt), du.to(dt)


def sparse_moe_block_ref(hidden, experts_indices, weights, eager_rounding: bool = True, acts=None):
    """SparseMoeBlock.forward (act.py:105-162).

    hidden [B, S, H]; experts_indices [B, S] (bool or integer expert id);
    weights = [(gate_w, up_w, down_w), ...] per expert (any number of experts);
    acts = each expert's `hidden_act` (default: silu for all).  Permute groups the rows
    by expert (stable), each expert runs on its contiguous row range
    [start_e, end_e) (act.py:142-154; ranges from act.py:1274-1283), rows of
    experts with no tokens stay zero (act.py:139), unpermute restores the order
    (probs are all ones and K == 1, so they have no effect, act.py:135,157).
    """
    from .permute import permute_ref, unpermute_ref, expert_offsets_ref

    B, S, H = hidden.shape
    x = hidden.reshape(-1, H)
    ids = experts_indices.reshape(-1)
    permuted, row_id_map, _ = permute_ref(x, ids)
    off = expert_offsets_ref(ids, len(weights)).tolist()
    out = torch.zeros_like(permuted)
    for e, (gw, uw, dw) in enumerate(weights):
        s, t = off[e], off[e + 1]
        if s == t:
            continue
        out[s:t] = swiglu_ffn_ref(permuted[s:t], gw, uw, dw, eager_rounding, "silu" if acts is None else acts[e])
    y = unpermute_ref(out, row_id_map)
    return y.view(B, S, H)
