"""GPU parity: token partition, permute, unpermute (bit-exact against the oracle), through the C ABI."""

import warnings

import pytest
import torch

import oracle
from wallx_mi355 import native, workloads as wl
from wallx_mi355.fusions import ops

pytestmark = pytest.mark.gpu


def _quiet(fn, *a, **k):
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        return fn(*a, **k)


@pytest.mark.parametrize("T,E,K,dtype", [
    (1, 2, 1, torch.bfloat16), (63, 2, 1, torch.float32), (64, 2, 1, torch.float16), (65, 2, 1, torch.bfloat16),
    (513, 3, 1, torch.bfloat16), (4096, 2, 1, torch.bfloat16), (1000, 4, 2, torch.float32),
    (777, 8, 3, torch.bfloat16), (2049, 200, 1, torch.float16),
])
def test_permute_unpermute_small(dev, T, E, K, dtype):
    g = torch.Generator().manual_seed(T + E + K)
    ids = torch.randint(0, E, (T, K) if K > 1 else (T,), generator=g, dtype=torch.int32)
    x = torch.randn(T, 64, generator=g).to(dtype)
    ref_p, ref_map, ref_sorted = oracle.permute_ref(x, ids)
    p, rmap = ops.permute(x.to(dev), ids.to(dev))
    assert rmap.dtype == torch.int32
    assert torch.equal(rmap.cpu(), ref_map)
    assert torch.equal(p.cpu(), ref_p)
    # sorted_row_id and offsets straight from the partition
    m2, off, srt, _ = native.partition(ids.to(dev), E, 0, None, want_sorted=True)
    assert torch.equal(m2.cpu(), ref_map) and torch.equal(srt.cpu(), ref_sorted)
    assert torch.equal(off.cpu(), oracle.expert_offsets_ref(ids, E))
    probs = torch.rand(T, K, generator=g) if K > 1 else None
    y = ops.unpermute(p, rmap, None if probs is None else probs.to(dev))
    assert torch.equal(y.cpu(), oracle.unpermute_ref(ref_p, ref_map, probs))


@pytest.mark.parametrize("id_dtype", [torch.bool, torch.int64, torch.int32])
def test_permute_accepts_reference_id_dtypes(dev, id_dtype):
    g = torch.Generator().manual_seed(2)
    types = torch.randint(0, 2, (3, 50), generator=g).to(id_dtype)
    x = torch.randn(150, 32, generator=g).to(torch.bfloat16)
    ref_p, ref_map, _ = oracle.permute_ref(x, types.reshape(-1))
    if id_dtype == torch.int32:
        p, rmap = ops.permute(x.to(dev), types.reshape(-1).to(dev))
    else:
        with pytest.warns(UserWarning, match="recommended type is torch.int32"):
            p, rmap = ops.permute(x.to(dev), types.reshape(-1).to(dev))
    assert torch.equal(rmap.cpu(), ref_map) and torch.equal(p.cpu(), ref_p)


def test_permute_num_out_tokens(dev):
    g = torch.Generator().manual_seed(4)
    ids = torch.randint(0, 3, (300,), generator=g, dtype=torch.int32)
    x = torch.randn(300, 16, generator=g)
    ref_p, ref_map, _ = oracle.permute_ref(x, ids, 200)
    p, rmap = ops.permute(x.to(dev), ids.to(dev), num_out_tokens=200)
    assert p.shape == (200, 16)
    assert torch.equal(rmap.cpu(), ref_map) and torch.equal(p.cpu(), ref_p)
    # without probs the op infers the token count from its input (ops.py:350), so pass them like the model does
    y = ops.unpermute(p, rmap, torch.ones(300, 1, device=dev))
    assert torch.equal(y.cpu(), oracle.unpermute_ref(ref_p, ref_map))  # dropped rows come back as zeros
    assert ops.unpermute(p, rmap).shape == (200, 16)


def test_out_of_range_ids_raise_the_status_word(dev):
    ids = torch.tensor([0, 5, 1, -1], dtype=torch.int32, device=dev)
    rmap, off, _, ws = native.partition(ids, 2, 0, None)
    assert int(ws[1].item()) == 1
    assert sorted(rmap.cpu().tolist()) == [0, 1, 2, 3]  # still a permutation
    rmap, off, _, ws = native.partition(torch.tensor([0, 1, 1, 0], dtype=torch.int32, device=dev), 2, 0, None)
    assert int(ws[1].item()) == 0 and off.cpu().tolist() == [0, 2, 4]


def test_config1_routing_is_identity(dev):
    x, types, _ = wl.config1()
    p, rmap = _quiet(ops.permute, x.view(-1, x.shape[-1]).to(dev), types.view(-1).to(dev))
    assert torch.equal(rmap.cpu(), torch.arange(512, dtype=torch.int32))
    assert torch.equal(p.cpu(), x.view(-1, x.shape[-1]))


def test_config3_full_size_properties(dev):
    """29184 x 2048 bf16: indices bit-exact against the oracle; rows checked through the round trip and
    the per-expert contiguity invariant."""
    x, types, _ = wl.config3()
    xf = x.view(-1, x.shape[-1]).to(dev)
    ids = types.view(-1)
    p, rmap = _quiet(ops.permute, xf, ids.to(dev))
    _, ref_map, _ = oracle.permute_ref(torch.zeros(ids.numel(), 1), ids)
    assert torch.equal(rmap.cpu(), ref_map)
    assert torch.equal(ops.unpermute(p, rmap), xf)                       # round trip is the identity
    n_vl = int((~ids).sum())
    assert n_vl == 28160
    assert torch.equal(p[:n_vl], xf[(~ids).to(dev)]) and torch.equal(p[n_vl:], xf[ids.to(dev)])


@pytest.mark.parametrize("T,H,n_act", [(300, 96, 37), (912, 2048, 32), (1000, 64, 1000), (70, 4096, 0), (515, 160, 200)])
def test_permute_rows_tiled_layout(dev, T, H, n_act):
    """The K-tiled activation matrix the FFN reads, decoded block by block on the host (16 x 32 blocks ordered
    [column block][row block], 16-byte chunk c of row r in slot c ^ ((r >> 2) & 3), each expert's rows starting at a
    multiple of 256, padding rows zero), against the rows in sorted order.  Both forms of the kernel (gather through
    the inverse map, with an odd and an even number of column blocks; scatter through row_id_map) bit for bit."""
    g = torch.Generator().manual_seed(T + H)
    x = torch.randn(T, H, generator=g).to(torch.bfloat16)
    types = torch.zeros(T, dtype=torch.bool)
    types[torch.randperm(T, generator=g)[:n_act]] = True
    rmap, off, inv, _ = native.partition(types.to(dev), 2, 0, None, want_sorted=True)
    rows_pad = native.padded_sorted_rows(T)
    n0 = T - n_act
    pad0 = (n0 + 255) // 256 * 256
    want = torch.zeros(rows_pad, H, dtype=torch.bfloat16)
    order = inv.cpu().long()
    want[:n0] = x[order[:n0]]
    want[pad0:pad0 + n_act] = x[order[n0:]]
    for form, tiled in (("gather", native.permute_rows_tiled(x.to(dev), rmap, off, None, inv)),
                        ("scatter", native.permute_rows_tiled(x.to(dev), rmap, off, None, None))):
        rb, kb = rows_pad // 16, H // 32
        t = tiled.cpu()[: rows_pad * H].view(kb, rb, 16, 4, 8)
        got = torch.empty(rows_pad, H, dtype=torch.bfloat16)
        for r in range(16):
            for c in range(4):
                got.view(rb, 16, kb, 4, 8)[:, r, :, c, :] = t[:, :, r, c ^ ((r >> 2) & 3), :].transpose(0, 1)
        live = torch.zeros(rows_pad, dtype=torch.bool)
        live[:n0] = True
        live[pad0:pad0 + n_act] = True
        assert torch.equal(got[live].view(torch.int16), want[live].view(torch.int16)), form
        if form == "gather":  # the gather form also zero-fills the padding rows
            assert torch.equal(got.view(torch.int16), want.view(torch.int16)), form


def test_one_million_tokens_round_trip(dev):
    """2^20 tokens x 1024 bf16 columns (2 GiB each way), eight experts, everything checked on the device through the
    properties the partition guarantees: the map is a permutation, rows of an expert are contiguous and in source
    order, offsets are the cumulative counts, and unpermute undoes permute bit for bit."""
    T, H, E = 1 << 20, 1024, 8
    g = torch.Generator(device=dev).manual_seed(1)
    x = torch.randint(-32768, 32767, (T, H), device=dev, generator=g, dtype=torch.int16).view(torch.bfloat16)
    ids = torch.randint(0, E, (T,), device=dev, generator=g, dtype=torch.int32)
    rmap, off, inv, _ = native.partition(ids, E, 0, None, want_sorted=True)
    counts = torch.bincount(ids.long(), minlength=E)
    assert torch.equal(off.long(), torch.cat([counts.new_zeros(1), counts.cumsum(0)]))
    assert torch.equal(torch.sort(rmap.long()).values, torch.arange(T, device=dev))
    assert torch.equal(inv.long()[rmap.long()], torch.arange(T, device=dev))          # inverse map
    sorted_ids = ids[inv.long()]
    assert bool((sorted_ids[1:] >= sorted_ids[:-1]).all())                             # experts contiguous, ascending
    same = sorted_ids[1:] == sorted_ids[:-1]
    assert bool((inv[1:][same] > inv[:-1][same]).all())                                # stable inside an expert
    p = native.permute_rows(x, rmap, 1, T)
    assert torch.equal(p.view(torch.int16), x.view(torch.int16)[inv.long()])
    back = native.unpermute(p, rmap, torch.tensor([]), T, 1)
    assert torch.equal(back.view(torch.int16), x.view(torch.int16))


def test_config4_skewed_groups(dev):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2048, 256, generator=g).to(torch.bfloat16).to(dev)
    ids = torch.ones(2048, dtype=torch.bool, device=dev)               # VL group empty
    rmap, off, _, _ = native.partition(ids, 2)
    assert off.cpu().tolist() == [0, 0, 2048] and torch.equal(rmap.cpu(), torch.arange(2048, dtype=torch.int32))
    for n_act in (0, 1, 8, 32, 64):
        ids = torch.cat([torch.zeros(4096, dtype=torch.bool), torch.ones(n_act, dtype=torch.bool)])
        rmap, off, _, _ = native.partition(ids.to(dev), 2)
        assert off.cpu().tolist() == [0, 4096, 4096 + n_act]
        assert torch.equal(rmap.cpu(), torch.arange(4096 + n_act, dtype=torch.int32))


def test_permute_autograd_and_unpermute_backward(dev):
    g = torch.Generator().manual_seed(6)
    T, K, H = 200, 2, 32
    ids = torch.randint(0, 4, (T, K), generator=g, dtype=torch.int32)
    x = torch.randn(T, H, generator=g)
    probs = torch.rand(T, K, generator=g)
    xd = x.to(dev).requires_grad_(True)
    pd = probs.to(dev).requires_grad_(True)
    p, rmap = ops.permute(xd, ids.to(dev))
    y = ops.unpermute(p * 2.0, rmap, pd)
    gy = torch.randn(T, H, generator=g)
    y.backward(gy.to(dev))
    # y[t] = 2 x[t] sum_k p[t,k]  =>  dx = 2 gy sum_k p, dp[t,k] = <gy[t], 2 x[t]>
    assert torch.allclose(xd.grad.cpu(), 2 * gy * probs.sum(1, keepdim=True), rtol=1e-5, atol=1e-5)
    exp_dp = (gy * 2 * x).sum(1, keepdim=True).expand(T, K)
    assert torch.allclose(pd.grad.cpu(), exp_dp, rtol=1e-4, atol=1e-4)
    # native backward against the oracle restatement, bf16
    yb = torch.randn(T * K, H, generator=g).to(torch.bfloat16)
    gb = torch.randn(T, H, generator=g).to(torch.bfloat16)
    _, ref_map, _ = oracle.permute_ref(x, ids)
    ag, pg = native.unpermute_bwd(gb.to(dev), yb.to(dev), ref_map.to(dev), probs.to(dev))
    rag, rpg, _ = oracle.unpermute_bwd_ref(gb, yb, ref_map, probs)
    assert torch.equal(ag.cpu(), rag)
    assert torch.allclose(pg.cpu(), rpg, rtol=1e-5, atol=1e-4)
