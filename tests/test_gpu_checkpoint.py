"""Checkpoint adapter end to end on the GPU: safetensors on disk -> load_expert_weights -> SparseMoeBlock forward on
the kernels, against the oracle evaluated on the very tensors that were written (both key conventions of the
reference: act.py:785-794 and the trainer's dense -> expert 0 renaming, qwen_vl_act_trainer.py:661-671)."""

import os

import pytest
import torch

import oracle
from wallx_mi355 import checkpoint, moe, native

pytestmark = pytest.mark.gpu

H, INTER = 256, (384, 128)


class _Cfg:
    experts = [{"hidden_size": H, "intermediate_size": INTER[0], "hidden_act": "silu"},
               {"hidden_size": H, "intermediate_size": INTER[1], "hidden_act": "silu"}]


def _write_checkpoint(tmp_path, n_layers, dense, seed):
    from safetensors.torch import save_file

    g = torch.Generator().manual_seed(seed)
    sd = {"model.embed_tokens.weight": torch.zeros(4, 8, dtype=torch.bfloat16)}
    for layer in range(n_layers):
        for e, inter in enumerate(INTER):
            if dense and e == 1:
                continue
            for proj, shape in (("gate", (inter, H)), ("up", (inter, H)), ("down", (H, inter))):
                key = (f"model.layers.{layer}.mlp.{proj}_proj.weight" if dense
                       else checkpoint.expert_weight_key(layer, e, proj))
                sd[key] = (torch.randn(shape, generator=g) * 0.05).to(torch.bfloat16)
    keys = sorted(sd)
    save_file({k: sd[k] for k in keys[::2]}, os.path.join(tmp_path, "model-00001-of-00002.safetensors"))
    save_file({k: sd[k] for k in keys[1::2]}, os.path.join(tmp_path, "model-00002-of-00002.safetensors"))
    return sd


def _close(got, ref):
    got, ref = got.float().cpu(), ref.float()
    err = (got - ref).abs()
    assert bool((err <= 2e-2 + 1e-2 * ref.abs()).all()), f"max err {float(err.max())}"


@pytest.mark.parametrize("dense", [False, True])
@pytest.mark.parametrize("pack_only", [False, True])
def test_checkpoint_to_block_forward(dev, tmp_path, dense, pack_only):
    sd = _write_checkpoint(tmp_path, 2, dense, seed=11 + dense)
    torch.manual_seed(3)
    blocks = {layer: moe.SparseMoeBlock(_Cfg(), 2).to(torch.bfloat16).to(dev) for layer in range(2)}
    init1 = {layer: [w.detach().clone().cpu() for w in blocks[layer].experts[1].weights()] for layer in blocks}
    # a forward BEFORE loading leaves packed copies of the initial weights behind: loading must not reuse them
    g = torch.Generator().manual_seed(5)
    x = torch.randn(2, 150, H, generator=g).to(torch.bfloat16)
    types = torch.rand(2, 150, generator=g) > 0.7
    with torch.no_grad():
        for b in blocks.values():
            b(x.to(dev), types.to(dev))
    counts = checkpoint.load_expert_weights(str(tmp_path), blocks, pack_only=pack_only)
    assert counts == ({0: 3, 1: 3} if dense else {0: 6, 1: 6})
    for layer, block in blocks.items():
        ws = []
        for e in range(2):
            if dense and e == 1:
                ws.append(tuple(init1[layer]))  # the action expert keeps its initialisation
            else:
                prefix = f"model.layers.{layer}.mlp." if dense else f"model.layers.{layer}.moe.experts.{e}."
                ws.append(tuple(sd[f"{prefix}{p}_proj.weight"] for p in ("gate", "up", "down")))
        ref = oracle.sparse_moe_block_ref(x, types, ws)
        with torch.no_grad():
            y = block(x.to(dev), types.to(dev))
        _close(y, ref)
        if pack_only:
            assert all(w.numel() == 0 for e in block.experts for w in e.weights())  # nn.Linear copies released
            assert sorted(n for n, _ in block.named_parameters()) == sorted(
                f"experts.{e}.{p}_proj.weight" for e in (0, 1) for p in ("gate", "up", "down"))
            with pytest.raises(RuntimeError, match="no backward"):
                block(x.to(dev).requires_grad_(True), types.to(dev))


def test_loading_into_a_block_that_kept_its_dense_weights_beside_the_packed_ones(dev):
    """pack_for_inference(free_dense=False) leaves a block with both forms; a later load must not leave it running the
    old packed weights."""
    torch.manual_seed(0)
    block = moe.SparseMoeBlock(_Cfg(), 2).to(torch.bfloat16).to(dev)
    block.pack_for_inference(free_dense=False)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(1, 120, H, generator=g).to(torch.bfloat16)
    types = torch.rand(1, 120, generator=g) > 0.5
    with torch.no_grad():
        before = block(x.to(dev), types.to(dev))
    sd = {}
    for e, inter in enumerate(INTER):
        for proj, shape in (("gate", (inter, H)), ("up", (inter, H)), ("down", (H, inter))):
            sd[checkpoint.expert_weight_key(0, e, proj)] = (torch.randn(shape, generator=g) * 0.05).to(torch.bfloat16)
    assert checkpoint.load_expert_weights(sd, {0: block}) == {0: 6}
    assert block._packed is not None  # packed again, from the new values
    with torch.no_grad():
        after = block(x.to(dev), types.to(dev))
    ws = [tuple(sd[checkpoint.expert_weight_key(0, e, p)] for p in ("gate", "up", "down")) for e in range(2)]
    _close(after, oracle.sparse_moe_block_ref(x, types, ws))
    assert int((after != before).sum()) > 0
    # a block whose dense copies were released has nothing to load into: refused, not silently skipped
    block.pack_for_inference(free_dense=True)
    with pytest.raises(ValueError, match="checkpoint shape"):
        checkpoint.load_expert_weights(sd, {0: block})


def test_weight_written_through_data_after_a_forward(dev):
    """`.data` writes do not move torch's version counter.  A block whose weights train repacks on every forward, so
    it sees them; a frozen block needs native.invalidate_packed()."""
    torch.manual_seed(0)
    block = moe.SparseMoeBlock(_Cfg(), 2).to(torch.bfloat16).to(dev)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(1, 200, H, generator=g).to(torch.bfloat16)
    types = torch.rand(1, 200, generator=g) > 0.5
    new_down = (torch.randn(H, INTER[0], generator=g) * 0.05).to(torch.bfloat16)

    def ref():
        ws = [tuple(w.detach().cpu() for w in e.weights()) for e in block.experts]
        return oracle.sparse_moe_block_ref(x, types, ws)

    y0 = block(x.to(dev), types.to(dev))                       # weights require grad: the training path
    _close(y0.detach(), ref())
    block.experts[0].down_proj.weight.data.copy_(new_down)     # master-weight / EMA style write
    y1 = block(x.to(dev), types.to(dev))
    _close(y1.detach(), ref())
    assert int((y1 != y0).sum()) > 0
    # frozen weights, no gradient tracking: the packed copies are cached ...
    for p in block.parameters():
        p.requires_grad_(False)
    with torch.no_grad():
        y2 = block(x.to(dev), types.to(dev))
        assert int((y2 != y1.detach()).sum()) == 0
        block.experts[0].down_proj.weight.copy_(2 * new_down)  # an in-place op on the tensor itself is seen
        y3 = block(x.to(dev), types.to(dev))
        _close(y3, ref())
        block.experts[1].up_proj.weight.data.mul_(0.5)         # invisible to the version counter ...
        native.invalidate_packed(block.experts[1].up_proj.weight)  # ... so the caller says so
        y4 = block(x.to(dev), types.to(dev))
        _close(y4, ref())
        assert int((y4 != y3).sum()) > 0


def test_routing_is_partitioned_once_for_all_layers(dev):
    """The reference's decoder passes the same moe_token_types tensor to every layer (act.py:257-261): the blocks
    share one partition as long as the tensor object and its contents stay the same."""
    torch.manual_seed(0)
    blocks = [moe.SparseMoeBlock(_Cfg(), 2).to(torch.bfloat16).to(dev) for _ in range(3)]
    g = torch.Generator().manual_seed(2)
    x = torch.randn(1, 300, H, generator=g).to(torch.bfloat16).to(dev)
    types = (torch.rand(1, 300, generator=g) > 0.6).to(dev)
    r = [b.route(types) for b in blocks]
    assert r[0] is r[1] is r[2]
    same_values = types.clone()
    assert blocks[0].route(same_values) is not r[0]            # another tensor object: partitioned again
    r1 = blocks[0].route(types)
    types[0, :5] = ~types[0, :5]                                # modified in place: partitioned again
    r2 = blocks[1].route(types)
    assert r2 is not r1
    ref_map = oracle.permute_ref(torch.zeros(300, 1), types.view(-1).cpu())[1]
    assert torch.equal(r2.row_id_map.cpu(), ref_map)
    with torch.no_grad():
        y = blocks[2](x, types)
    ws = [tuple(w.detach().cpu() for w in e.weights()) for e in blocks[2].experts]
    _close(y, oracle.sparse_moe_block_ref(x.cpu(), types.cpu(), ws))
