"""Oracle: modality-routed token permute / unpermute (test infrastructure only).

Follows the definition of ``row_id_map`` in the reference's native op
(csrc/permute.cu:39-67, 450-504) and the Python wrapper (ops.py:175-256,
284-392): a *stable* sort of the flattened ``indices[T, K]`` by expert id,
``row_id_map[k*T + t]`` = sorted position of source row ``t*K + k`` (or -1
when that position is >= ``num_out_tokens``), ``permuted[p] = x[src(p) // K]``.
"""

import torch


def _as_2d_ids(indices: torch.Tensor) -> torch.Tensor:
    # ops.py:197-199 -- top-1 ids are viewed as [T, 1]
    ids = indices.view(-1, 1) if indices.dim() == 1 else indices
    return ids.to(torch.int32)  # ops.py:219-224


def permute_ref(x: torch.Tensor, indices: torch.Tensor, num_out_tokens: int = 0):
    """Returns (permuted [num_out, H], row_id_map [T*K] int32, sorted_row_id [T*K] int32).

    csrc/permute.cu:472-494 sorts (key = expert id, value = flat row id) with a
    stable radix sort; torch.argsort(stable=True) is the library routine with the
    same contract.  csrc/permute.cu:496-504: num_out_tokens <= 0 means "all".
    """
    ids = _as_2d_ids(indices)
    T, K = ids.shape
    n = T * K
    flat = ids.reshape(-1)
    sorted_row_id = torch.argsort(flat, stable=True).to(torch.int32)  # position -> t*K+k
    num_out = num_out_tokens if num_out_tokens and num_out_tokens > 0 else n
    pos = torch.arange(n, dtype=torch.int32)
    src_tok = (sorted_row_id // K).long()
    src_k = (sorted_row_id % K).long()
    row_id_map = torch.empty(n, dtype=torch.int32)
    # csrc/permute.cu:56-66
    row_id_map[src_k * T + src_tok] = torch.where(pos < num_out, pos, torch.full_like(pos, -1))
    permuted = x[src_tok[:num_out]].clone()  # csrc/permute.cu:156-262 (forward branch)
    return permuted, row_id_map, sorted_row_id


def expert_offsets_ref(indices: torch.Tensor, num_experts: int) -> torch.Tensor:
    """[E+1] int32 exclusive prefix of per-expert row counts.

    Restates the caller's bookkeeping act.py:1274-1283 (group_size, cumsum,
    start = cumsum - size, end = cumsum) as one offsets vector.
    """
    flat = _as_2d_ids(indices).reshape(-1).long()
    counts = torch.bincount(flat, minlength=num_experts)[:num_experts]
    off = torch.zeros(num_experts + 1, dtype=torch.int32)
    off[1:] = torch.cumsum(counts, 0).to(torch.int32)
    return off


def _round_to(v: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    return v.to(dtype).to(torch.float32)


def unpermute_ref(y: torch.Tensor, row_id_map: torch.Tensor, probs: torch.Tensor = None,
                  num_tokens: int = None, num_topk: int = None):
    """out[t] = sum_k prob[t,k] * y[row_id_map[k*T+t]], skipping -1 rows.

    csrc/permute.cu:405-415 dispatches hasProb=false whenever topK == 1, so with
    K == 1 the probabilities are ignored and the op is a pure row gather (rows
    mapped to -1 come out as zeros, csrc/permute.cu:120-123).  For K > 1 the
    kernel multiplies and accumulates in its compute type (bf16 for bf16 input,
    csrc/permute.cu:700-720), one rounding per operation, in k order.
    """
    rid = row_id_map.long()
    if probs is not None and probs.numel():
        T, K = probs.shape
    else:
        K = num_topk or 1
        T = num_tokens if num_tokens is not None else rid.numel() // K
    H = y.shape[1]
    ct = y.dtype  # compute type == storage type in the reference kernels
    out = torch.zeros(T, H, dtype=torch.float32)
    use_prob = probs is not None and probs.numel() > 0 and K > 1
    for k in range(K):
        r = rid[k * T:(k + 1) * T]
        valid = r >= 0
        rows = torch.zeros(T, H, dtype=torch.float32)
        rows[valid] = y[r[valid]].to(torch.float32)
        if use_prob:
            p = _round_to(probs[:, k:k + 1].to(torch.float32), ct)
            rows = _round_to(rows * p, ct)
        if k == 0:
            out = rows
        else:
            summed = _round_to(out + rows, ct)
            # csrc/permute.cu:131-132: a -1 row is skipped (no add, no rounding)
            out = torch.where(valid[:, None], summed, out)
    return out.to(y.dtype)


def unpermute_bwd_ref(grad_out: torch.Tensor, y_fwd: torch.Tensor, row_id_map: torch.Tensor,
                      probs: torch.Tensor):
    """Backward of unpermute (csrc/permute.cu:156-262 with input_fwd != null,
    781-942): act_grad[row_id_map[k*T+t]] = grad_out[t] * prob[t,k] (no prob
    factor when K == 1), prob_grad[t,k] = <grad_out[t], y_fwd[row]> in fp32.
    Rows of act_grad that no token maps to are left unwritten by the kernel
    (torch::empty); the oracle reports them as zeros and returns the written mask.
    """
    T, K = probs.shape
    rid = row_id_map.long()
    n_rows = y_fwd.shape[0]
    ct = grad_out.dtype
    act_grad = torch.zeros(n_rows, grad_out.shape[1], dtype=torch.float32)
    written = torch.zeros(n_rows, dtype=torch.bool)
    prob_grad = torch.zeros(T, K, dtype=torch.float32)
    g = grad_out.to(torch.float32)
    for k in range(K):
        r = rid[k * T:(k + 1) * T]
        valid = r >= 0
        if K > 1:
            p = _round_to(probs[:, k:k + 1].to(torch.float32), ct)
            val = _round_to(g * p, ct)
        else:
            val = g
        act_grad[r[valid]] = val[valid]
        written[r[valid]] = True
        if K > 1:
            yf = torch.zeros(T, y_fwd.shape[1], dtype=torch.float32)
            yf[valid] = y_fwd[r[valid]].to(torch.float32)
            # products are formed in the compute type, summed in fp32
            prob_grad[:, k] = _round_to(g * yf, ct).sum(1)
    return act_grad.to(grad_out.dtype), prob_grad, written
