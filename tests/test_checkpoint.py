"""Checkpoint adapter (CPU): the reference's key conventions (act.py:785-794, qwen_vl_act_trainer.py:657-671) map
onto SparseMoeBlock parameters; safetensors files are read tensor by tensor."""

import os

import pytest
import torch

from wallx_mi355 import checkpoint, moe


class _Cfg:
    experts = [{"hidden_size": 64, "intermediate_size": 96, "hidden_act": "silu"},
               {"hidden_size": 64, "intermediate_size": 32, "hidden_act": "silu"}]


def _blocks(n):
    return {layer: moe.SparseMoeBlock(_Cfg(), 2).to(torch.bfloat16) for layer in range(n)}


def _state(n, dense=False, seed=0):
    g = torch.Generator().manual_seed(seed)
    sd = {"model.embed_tokens.weight": torch.zeros(3, 4)}
    for layer in range(n):
        for e, cfg in enumerate(_Cfg.experts):
            if dense and e == 1:
                continue
            for proj, shape in (("gate", (cfg["intermediate_size"], 64)), ("up", (cfg["intermediate_size"], 64)),
                                ("down", (64, cfg["intermediate_size"]))):
                key = (f"model.layers.{layer}.mlp.{proj}_proj.weight" if dense
                       else checkpoint.expert_weight_key(layer, e, proj))
                sd[key] = torch.randn(shape, generator=g).to(torch.bfloat16)
    return sd


def test_key_classification():
    assert checkpoint.classify_key("model.layers.7.moe.experts.1.down_proj.weight") == (7, 1, "down")
    assert checkpoint.classify_key("model.layers.3.mlp.gate_proj.weight") == (3, 0, "gate")
    assert checkpoint.classify_key("model.layers.3.mlp.gate_proj.weight", dense_as_expert0=False) is None
    assert checkpoint.classify_key("model.layers.3.self_attn.q_proj.weight") is None
    assert checkpoint.classify_key("visual.blocks.3.mlp.gate_proj.weight") is None  # the vision tower's MLPs


def test_load_from_state_dict_and_from_safetensors(tmp_path):
    from safetensors.torch import save_file

    sd = _state(2)
    blocks = _blocks(2)
    counts = checkpoint.load_expert_weights(sd, blocks)
    assert counts == {0: 6, 1: 6}
    assert torch.equal(blocks[1].experts[1].up_proj.weight, sd[checkpoint.expert_weight_key(1, 1, "up")])
    # two shards on disk
    keys = sorted(sd)
    save_file({k: sd[k] for k in keys[: len(keys) // 2]}, os.path.join(tmp_path, "model-00001-of-00002.safetensors"))
    save_file({k: sd[k] for k in keys[len(keys) // 2:]}, os.path.join(tmp_path, "model-00002-of-00002.safetensors"))
    fresh = _blocks(2)
    assert checkpoint.load_expert_weights(str(tmp_path), fresh) == {0: 6, 1: 6}
    for layer in range(2):
        for e in range(2):
            for a, b in zip(fresh[layer].experts[e].weights(), blocks[layer].experts[e].weights()):
                assert torch.equal(a, b)


def test_dense_checkpoint_fills_the_vl_expert_only():
    sd = _state(1, dense=True)
    blocks = _blocks(1)
    before = blocks[0].experts[1].gate_proj.weight.detach().clone()
    assert checkpoint.load_expert_weights(sd, blocks) == {0: 3}
    assert torch.equal(blocks[0].experts[0].down_proj.weight, sd["model.layers.0.mlp.down_proj.weight"])
    assert torch.equal(blocks[0].experts[1].gate_proj.weight, before)


def test_errors():
    blocks = _blocks(1)
    sd = _state(1)
    bad = dict(sd)
    bad[checkpoint.expert_weight_key(0, 0, "gate")] = torch.zeros(5, 5)
    with pytest.raises(ValueError, match="checkpoint shape"):
        checkpoint.load_expert_weights(bad, blocks)
    short = {k: v for k, v in sd.items() if "experts.1.down" not in k}
    with pytest.raises(KeyError, match="expert 1"):
        checkpoint.load_expert_weights(short, blocks)
    with pytest.raises(FileNotFoundError):
        checkpoint.load_expert_weights("/nonexistent/dir", blocks)


def test_strict_moe_checkpoint_must_hold_both_experts_and_params_must_be_bf16():
    sd = _state(1)
    only0 = {k: v for k, v in sd.items() if "experts.1." not in k}  # MoE key names, expert 1 absent altogether
    with pytest.raises(KeyError, match="expert 1"):
        checkpoint.load_expert_weights(only0, _blocks(1))
    assert checkpoint.load_expert_weights(only0, _blocks(1), strict=False) == {0: 3}
    fp32_block = {0: moe.SparseMoeBlock(_Cfg(), 2)}
    with pytest.raises(TypeError, match="bfloat16"):
        checkpoint.load_expert_weights(sd, fp32_block)
