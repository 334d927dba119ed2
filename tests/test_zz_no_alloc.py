"""The allocation-free partition entry point (wx_partition_build_noalloc: histograms in a device array built into the
library) against wx_partition_build through the C ABI: bit-equal row_id_map, inverse map and expert offsets, on
two calls in a row, the second with a smaller input (the built-in array keeps the first call's contents)."""

import pytest
import torch

from wallx_mi355 import _lib

pytestmark = pytest.mark.gpu


def _both(ids, num_experts, topk, num_out, dev):
    ids = ids.to(dev)
    T = ids.shape[0]
    n = T * topk
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for entry in ("wx_partition_build", "wx_partition_build_noalloc"):
        rmap = torch.full((n,), -7, dtype=torch.int32, device=dev)
        srt = torch.full((n,), -7, dtype=torch.int32, device=dev)
        off = torch.full((num_experts + 1,), -7, dtype=torch.int32, device=dev)
        status = torch.zeros(1, dtype=torch.int32, device=dev)
        args = [ids.data_ptr(), _lib.WX_I32, T, topk, num_experts, num_out, rmap.data_ptr(), srt.data_ptr(),
                off.data_ptr(), status.data_ptr()]
        if entry == "wx_partition_build":
            nbytes = _lib.load().wx_partition_workspace_bytes(n)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            args += [ws.data_ptr(), nbytes]
        _lib.call(entry, *args, stream)
        torch.cuda.synchronize()
        outs.append((rmap.cpu(), srt.cpu(), off.cpu(), status.cpu()))
    return outs


def test_noalloc_partition_equals_the_workspace_entry_point_twice_in_a_row(dev):
    g = torch.Generator().manual_seed(7)
    # first a large call (600 000 expanded tokens: more than 1024 segments' worth, so the segment length grows),
    # then smaller ones: 100 000 keys reuse the same built-in array; the last three are small enough for the
    # single-workgroup form of the partition, which needs no histogram buffer at all
    for T, E, K, num_out in ((300000, 7, 2, 0), (100000, 5, 1, 0), (29184, 2, 1, 0), (513, 200, 3, 1000), (1, 2, 1, 0)):
        ids = torch.randint(0, E, (T, K), generator=g, dtype=torch.int32)
        (m0, s0, o0, st0), (m1, s1, o1, st1) = _both(ids, E, K, num_out, dev)
        assert torch.equal(m0, m1), f"row_id_map differs at T={T}"
        assert torch.equal(s0, s1), f"sorted_row_id differs at T={T}"
        assert torch.equal(o0, o1) and int(st0) == int(st1) == 0
        # and both are the stable partition (a permutation whose inverse groups the ids in order)
        flat = ids.reshape(-1)
        assert torch.equal(flat[s1.long()], torch.sort(flat, stable=True).values)


def test_noalloc_init_is_idempotent(dev):
    lib = _lib.load()
    assert lib.wx_partition_noalloc_init() == 0
    assert lib.wx_partition_noalloc_init() == 0


def test_noalloc_partition_rejects_what_does_not_fit(dev):
    lib = _lib.load()
    p = torch.zeros(8, dtype=torch.int32, device=dev).data_ptr()
    assert lib.wx_partition_build_noalloc(p, _lib.WX_I32, 2 ** 31, 1, 2, 0, p, p, p, None, None) == -2
    assert b"2^31-1" in lib.wx_last_error_string()
    assert lib.wx_partition_build_noalloc(p, _lib.WX_I32, 4, 129, 2, 0, p, p, p, None, None) == -2
