"""Writes the golden fixtures under tests/golden/ from the CPU oracle on the seeded BASELINE inputs.

    python tests/golden/make_golden.py

The reference has no tests, fixtures or golden vectors of its own, and its Python package is not importable in
this environment, so these vectors come from the oracle (oracle/), which restates the reference's PyTorch path
and is pinned separately by tests/test_oracle_*.py.  The fixtures freeze the oracle's results so that a later
change of the oracle or of the input generators is noticed, and give the GPU tests fixed targets.
Files are small .npz archives (integers in full, floating-point outputs as row samples).
"""

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, os.path.join(ROOT, "wall-x_amd"))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from wallx_mi355 import workloads as wl  # noqa: E402


def bf16_bits(t):
    return t.contiguous().view(torch.int16).numpy()


def config1():
    x, types, ws = wl.config1()
    xf = x.view(-1, x.shape[-1])
    permuted, rmap, _ = oracle.permute_ref(xf, types.view(-1))
    y = oracle.sparse_moe_block_ref(x, types, [w.as_tuple() for w in ws])[0]
    g = torch.Generator().manual_seed(1)
    rows = torch.cat([torch.tensor([0, 1, 447, 448, 511]), torch.randperm(512, generator=g)[:27]]).sort().values
    np.savez_compressed(os.path.join(HERE, "config1_moe_layer_fp32.npz"),
                        row_id_map=rmap.numpy(), rows=rows.numpy(), out_rows=y[rows].numpy(),
                        out_row_sums=y.double().sum(1).numpy(), out_row_abs_sums=y.double().abs().sum(1).numpy(),
                        permuted_row_sums=permuted.double().sum(1).numpy())


def config2():
    ids, grid = wl.config2_tokens()
    pos, delta = oracle.rope_index_ref(ids, 2, wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, 2,
                                       image_grid_thw=grid)
    rot_ids = oracle.rot_pos_ids_ref(grid, 2)
    table = oracle.rot_pos_emb_ref(wl.vision_inv_freq(), grid, 2)
    wi, cu = oracle.window_index_dedup_ref(grid, 112, 2, 14, 4)
    cos, sin = oracle.rotary_cos_sin_ref(pos, wl.text_inv_freq(), torch.bfloat16)
    q, k = wl.qk_inputs(16, 896)
    qo, ko = oracle.mrope_apply_ref(q.transpose(1, 2), k.transpose(1, 2), cos, sin, list(wl.MROPE_SECTION))
    toks = torch.tensor([0, 10, 11, 12, 27, 268, 300, 783, 784, 895])
    np.savez_compressed(os.path.join(HERE, "config2_positions_and_rope.npz"),
                        position_ids=pos.numpy().astype(np.int16), mrope_deltas=delta.numpy(),
                        rot_pos_ids=rot_ids.numpy().astype(np.int16), rot_pos_table_rows=table[:1024:37].numpy(),
                        rot_pos_table_sum=np.float64(table.double().sum().item()),
                        window_index=wi.numpy(), cu_window_seqlens=cu.numpy(),
                        rope_tokens=toks.numpy(), rope_batches=np.array([0, 15]),
                        q_out=bf16_bits(qo[[0, 15]][:, :, toks]), k_out=bf16_bits(ko[[0, 15]][:, :, toks]))


def config3():
    x, types, ws = wl.config3()
    T = x.shape[0] * x.shape[1]
    xf, tf = x.view(T, -1), types.view(T)
    _, rmap, _ = oracle.permute_ref(torch.zeros(T, 1), tf)
    off = oracle.expert_offsets_ref(tf, 2)
    g = torch.Generator().manual_seed(1)
    act_rows, vl_rows = torch.nonzero(tf).flatten(), torch.nonzero(~tf).flatten()
    pick = torch.cat([vl_rows[torch.randperm(vl_rows.numel(), generator=g)[:40]], vl_rows[:2], vl_rows[-2:],
                      act_rows[torch.randperm(act_rows.numel(), generator=g)[:12]], act_rows[:2], act_rows[-2:]])
    y = oracle.sparse_moe_block_ref(xf[pick][None], tf[pick][None], [w.as_tuple() for w in ws])[0]
    np.savez_compressed(os.path.join(HERE, "config3_moe_layer_bf16.npz"),
                        row_id_map=rmap.numpy(), expert_offsets=off.numpy(), rows=pick.numpy(), out_rows=bf16_bits(y))


if __name__ == "__main__":
    torch.set_num_threads(8)
    config1()
    config2()
    config3()
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")
