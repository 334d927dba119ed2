"""GPU parity: rope_index, rot_pos_emb, get_window_index -- integer outputs, bit-exact against the oracle."""

import pytest
import torch

import oracle
from wallx_mi355 import native, workloads as wl
from wallx_mi355.fusions import ops

pytestmark = pytest.mark.gpu

I, V, S0, E0, TX = wl.IMAGE_TOKEN_ID, wl.VIDEO_TOKEN_ID, wl.VISION_START_TOKEN_ID, wl.VISION_END_TOKEN_ID, wl.TEXT_TOKEN_ID


def _rope_both(dev, ids, tps=2, ig=None, vg=None, spg=None, mask=None):
    ref = oracle.rope_index_ref(ids, 2, I, V, S0, tps, ig, vg, spg, mask)
    mv = lambda t: None if t is None else t.to(dev)
    got = ops.get_rope_index(ids.to(dev), 2, I, V, S0, tps, mv(ig), mv(vg), mv(spg), mv(mask))
    assert got[0].dtype == torch.int64 and got[1].dtype == torch.int64
    assert got[0].shape == ref[0].shape and got[1].shape == ref[1].shape
    assert torch.equal(got[0].cpu(), ref[0]), "position_ids differ"
    assert torch.equal(got[1].cpu(), ref[1]), "deltas differ"
    return got


def test_rope_index_config2(dev):
    ids, grid = wl.config2_tokens()
    pos, delta = _rope_both(dev, ids, ig=grid)
    assert int(pos.max()) == 175 and delta.cpu().tolist() == [[-720]] * 16


def test_rope_index_reference_docstring_vector(dev):
    ids = torch.tensor([[S0] + [V] * 12 + [TX] * 5])
    pos, _ = _rope_both(dev, ids, tps=25, vg=torch.tensor([[3, 4, 4]]), spg=torch.tensor([2.0]))
    assert (pos[0, 0, 1:13] - 1).cpu().tolist() == [0] * 4 + [50] * 4 + [100] * 4


def test_rope_index_text_only_branches(dev):
    g = torch.Generator().manual_seed(1)
    ids = torch.randint(0, 1000, (5, 77), generator=g)
    _rope_both(dev, ids)
    mask = (torch.rand(5, 77, generator=g) > 0.3).long()
    mask[3] = 0
    _rope_both(dev, ids, mask=mask)


def _random_rows(g, B, S, n_items, video=False):
    """Rows with random text gaps, images (and videos), right- or left-padded to S."""
    rows, masks, igs, vgs, spgs = [], [], [], [], []
    for b in range(B):
        row = []
        for _ in range(int(torch.randint(0, n_items + 1, (1,), generator=g))):
            row += [TX] * int(torch.randint(0, 9, (1,), generator=g))
            t = int(torch.randint(1, 4, (1,), generator=g)) if video else 1
            h = 2 * int(torch.randint(1, 5, (1,), generator=g))
            w = 2 * int(torch.randint(1, 5, (1,), generator=g))
            is_vid = video and bool(torch.randint(0, 2, (1,), generator=g))
            row += [S0] + [V if is_vid else I] * (t * (h // 2) * (w // 2)) + [E0]
            if is_vid:
                vgs.append([t, h, w])
                spgs.append(float(torch.rand(1, generator=g)) * 3)
            else:
                igs.append([t, h, w])
        row += [TX] * int(torch.randint(1, 20, (1,), generator=g))
        assert len(row) <= S
        pad = S - len(row)
        if b % 2:
            rows.append([0] * pad + row); masks.append([0] * pad + [1] * len(row))
        else:
            rows.append(row + [0] * pad); masks.append([1] * len(row) + [0] * pad)
    ig = torch.tensor(igs).reshape(-1, 3)
    vg = torch.tensor(vgs).reshape(-1, 3) if vgs else None
    spg = torch.tensor(spgs) if spgs else None
    return torch.tensor(rows), torch.tensor(masks), ig, vg, spg


@pytest.mark.parametrize("seed,video", [(0, False), (1, False), (2, True), (3, True), (4, True)])
def test_rope_index_random_layouts_with_padding(dev, seed, video):
    g = torch.Generator().manual_seed(seed)
    ids, mask, ig, vg, spg = _random_rows(g, 6, 400, 5, video)
    _rope_both(dev, ids, tps=2.5 if video else 2, ig=ig, vg=vg, spg=spg, mask=mask)


def test_rope_index_many_images_per_row(dev):
    """More vision items in one row than one LDS batch of descriptors (and than the reference kernel's cap of 64)."""
    n = 300
    row = []
    for _ in range(n):
        row += [TX, S0, I, I, E0]
    row += [TX] * 7
    ids = torch.tensor([row, row])
    grid = torch.tensor([[1, 2, 4]] * (2 * n))
    _rope_both(dev, ids, ig=grid)


@pytest.mark.parametrize("S", [20000, 30720, 30721, 65536])
def test_rope_index_long_rows(dev, S):
    """Long rows (thousands of images between short text runs, a masked tail on one row): up to 30 720 tokens the
    compacted row stays in LDS (above 48 KiB of it with a raised limit), beyond that in the workspace."""
    g = torch.Generator().manual_seed(5)
    rows, masks, n_images = [], [], 0
    for b in range(2):
        valid = S - 40 * b  # the second row ends in 40 masked positions
        row = []
        while len(row) + 13 <= valid - 5:
            row += [TX] * int(torch.randint(0, 4, (1,), generator=g)) + [S0] + [I] * 8 + [E0]
            n_images += 1
        row += [TX] * (valid - len(row))
        rows.append(row + [TX] * (S - valid))
        masks.append([1] * valid + [0] * (S - valid))
    ids = torch.tensor(rows)
    grid = torch.tensor([[1, 4, 8]] * n_images)
    _rope_both(dev, ids, ig=grid, mask=torch.tensor(masks))


def test_rope_index_malformed_row_sets_status(dev):
    ids = torch.tensor([[TX, S0, I, I, TX]], device=dev)
    # the grid claims 4 merged tokens but the row ends after 3: the PyTorch path builds 6 positions for 5 tokens
    with pytest.raises(oracle.rope_index.RopeIndexInputError):
        oracle.rope_index_ref(ids.cpu(), 2, I, V, S0, 2, image_grid_thw=torch.tensor([[1, 4, 4]]))
    _, _, status = native.rope_index(ids, torch.tensor([[1, 4, 4]], device=dev), None, None, None, 2, I, V, S0, 2.0,
                                     return_status=True)
    assert int(status.item()) == 1
    ids = torch.tensor([[TX, S0, I, I, I, I, TX]], device=dev)
    _, _, status = native.rope_index(ids, torch.tensor([[1, 4, 4]], device=dev), None, None, None, 2, I, V, S0, 2.0,
                                     return_status=True)
    assert int(status.item()) == 0


GRIDS = [
    [(1, 32, 32)] * 48,
    [(1, 4, 4)],
    [(2, 10, 14), (1, 6, 22), (3, 18, 8)],
    [(1, 2, 2), (1, 34, 46), (1, 8, 8)],
    [(1, 70, 36)],
]


@pytest.mark.parametrize("grids", GRIDS)
@pytest.mark.parametrize("gdtype", [torch.int32, torch.int64])
def test_rot_pos_emb(dev, grids, gdtype):
    grid = torch.tensor(grids, dtype=gdtype)
    inv = wl.vision_inv_freq()
    ref = oracle.rot_pos_emb_ref(inv, grid, 2)
    got = ops.rot_pos_emb(inv.to(dev), grid.to(dev), 2)
    assert got.dtype == torch.float32 and got.shape == ref.shape
    assert torch.equal(got.cpu(), ref)  # one fp32 product per entry: bit-exact
    got2, ids = native.rot_pos_emb(inv.to(dev), grid.to(dev), 2, grid_thw_host=grid, return_ids=True)
    assert torch.equal(got2.cpu(), ref) and torch.equal(ids.cpu(), oracle.rot_pos_ids_ref(grid, 2))


def test_rot_pos_emb_odd_frequency_count_and_merge3(dev):
    inv = torch.rand(7)
    grid = torch.tensor([[2, 6, 9], [1, 3, 3]])
    assert torch.equal(ops.rot_pos_emb(inv.to(dev), grid.to(dev), 3).cpu(), oracle.rot_pos_emb_ref(inv, grid, 3))


@pytest.mark.parametrize("grids", GRIDS)
def test_window_index(dev, grids):
    grid = torch.tensor(grids)
    ref_wi, ref_cu = oracle.window_index_dedup_ref(grid, 112, 2, 14, 4)
    wi, cu = ops.get_window_index(grid.to(dev), 112, 2, 14, 4)
    assert wi.dtype == torch.int32 and cu.dtype == torch.int32
    assert torch.equal(wi.cpu(), ref_wi) and torch.equal(cu.cpu(), ref_cu)
    # same result from a CPU grid (moved by the op) and with an explicit host copy
    wi2, cu2 = ops.get_window_index(grid, 112, 2, 14, 4)
    assert torch.equal(wi2.cpu(), ref_wi) and torch.equal(cu2.cpu(), ref_cu)


def test_window_index_other_window_sizes_and_empty(dev):
    grid = torch.tensor([[1, 26, 18], [2, 12, 40]])
    for window, unit in ((56, 4), (168, 1), (112, 9)):
        ref_wi, ref_cu = oracle.window_index_dedup_ref(grid, window, 2, 14, unit)
        wi, cu = ops.get_window_index(grid.to(dev), window, 2, 14, unit)
        assert torch.equal(wi.cpu(), ref_wi) and torch.equal(cu.cpu(), ref_cu)
    wi, cu = ops.get_window_index(torch.zeros(0, 3, dtype=torch.int32, device=dev), 112, 2, 14, 4)
    assert wi.numel() == 0 and cu.cpu().tolist() == [0]
