"""Expert weights of a wall-x checkpoint -> `wallx_mi355.moe.SparseMoeBlock` modules.

The reference stores its weights as safetensors files in the model directory and loads every tensor into one
state dict (act.py:785-794).  Expert e of decoder layer L lives under
``model.layers.{L}.moe.experts.{e}.{gate,up,down}_proj.weight``; when training starts from a dense Qwen2.5-VL
checkpoint, the trainer renames ``model.layers.{L}.mlp.*`` to ``...moe.experts.0.*`` and leaves the action expert at
its initialisation (qwen_vl_act_trainer.py:657-671).  Both conventions are handled here.

Only safetensors are read (no pickles are ever loaded), one tensor at a time, so a multi-file checkpoint never
sits in host memory as a whole.
"""

import glob
import os
import re
from typing import Dict, Iterable, Mapping, Optional

import torch

_EXPERT_KEY = re.compile(r"(?:^|\.)layers\.(\d+)\.moe\.experts\.(\d+)\.(gate|up|down)_proj\.weight$")
_DENSE_KEY = re.compile(r"(?:^|\.)layers\.(\d+)\.mlp\.(gate|up|down)_proj\.weight$")


def expert_weight_key(layer: int, expert: int, proj: str, prefix: str = "model.") -> str:
    return f"{prefix}layers.{layer}.moe.experts.{expert}.{proj}_proj.weight"


def classify_key(key: str, dense_as_expert0: bool = True):
    """(layer, expert, proj) for a key that holds an expert projection weight, else None."""
    m = _EXPERT_KEY.search(key)
    if m:
        return int(m.group(1)), int(m.group(2)), m.group(3)
    if dense_as_expert0:
        m = _DENSE_KEY.search(key)
        if m:
            return int(m.group(1)), 0, m.group(2)
    return None


def iter_safetensors(path: str) -> Iterable:
    """Yields (key, tensor) over every *.safetensors file of a directory (or over one file)."""
    from safetensors import safe_open

    files = [path] if os.path.isfile(path) else sorted(glob.glob(os.path.join(path, "*.safetensors")))
    if not files:
        raise FileNotFoundError(f"no safetensors files under {path}")
    for f in files:
        with safe_open(f, framework="pt", device="cpu") as handle:
            for key in handle.keys():
                yield key, handle.get_tensor(key)


def load_expert_weights(source, blocks: Mapping[int, torch.nn.Module], dense_as_expert0: bool = True,
                        strict: bool = True, pack_only: bool = False) -> Dict[int, int]:
    """Copies expert projection weights into `blocks` (decoder layer index -> SparseMoeBlock).

    source: a checkpoint directory / safetensors file, or an already loaded state dict.
    Returns {layer: number of tensors loaded}.  With strict=True a layer for which the checkpoint holds any
    ``moe.experts.*`` key must receive all six tensors; a layer that only has dense ``mlp.*`` keys must receive
    expert 0's three (the action expert then keeps its initialisation, as in the trainer).  Shapes are checked, and
    so is the dtype of the block's parameters: the kernels are bf16 only.  Cached K-tiled copies of the touched
    parameters are dropped, so the next forward packs the new values.  A block that was packed for inference with
    its nn.Linear copies kept (`pack_for_inference(free_dense=False)`) would go on running its old packed weights:
    its packed set is dropped before the copy and rebuilt from the new values at the end.  A block whose nn.Linear
    copies were released cannot be loaded into (its parameters are empty: the shape check raises).
    pack_only=True finishes with `block.pack_for_inference()` on every block: the weights are packed into the
    K-tiled layout and the nn.Linear copies released (forward-only blocks, half the expert memory).
    """
    from . import native

    items = source.items() if isinstance(source, Mapping) else iter_safetensors(source)
    loaded: Dict[int, set] = {layer: set() for layer in blocks}
    moe_format: Dict[int, bool] = {layer: False for layer in blocks}
    repack = set()  # layers whose block held a packed set next to its nn.Linear copies
    for layer, block in blocks.items():
        for e in block.experts:
            for w in e.weights():
                if w.dtype != torch.bfloat16:
                    raise TypeError(f"layer {layer}: expert parameters are {w.dtype}; the kernels need torch.bfloat16 "
                                    "(call block.to(torch.bfloat16) before loading)")
    for key, tensor in items:
        hit = classify_key(key, dense_as_expert0)
        if hit is None:
            continue
        layer, expert, proj = hit
        block = blocks.get(layer)
        if block is None:
            continue
        if _EXPERT_KEY.search(key):
            moe_format[layer] = True
        if expert >= len(block.experts):
            continue
        param = getattr(block.experts[expert], f"{proj}_proj").weight
        if tuple(param.shape) != tuple(tensor.shape):
            raise ValueError(f"{key}: checkpoint shape {tuple(tensor.shape)} != module shape {tuple(param.shape)}")
        if getattr(block, "_packed", None) is not None:
            block._packed = None  # built from the values about to be overwritten
            repack.add(layer)
        with torch.no_grad():
            param.copy_(tensor.to(device=param.device, dtype=param.dtype))
        native.invalidate_packed(param)
        loaded[layer].add((expert, proj))
    if strict:
        for layer, got in loaded.items():
            must = range(len(blocks[layer].experts)) if moe_format[layer] else (0,)
            for e in must:
                missing = {"gate", "up", "down"} - {p for ee, p in got if ee == e}
                if missing:
                    raise KeyError(f"layer {layer}, expert {e}: missing {sorted(missing)} projection weights")
    if pack_only:
        for block in blocks.values():
            block.pack_for_inference(free_dense=True)
    else:
        for layer in sorted(repack):
            blocks[layer].pack_for_inference(free_dense=False)
    return {layer: len(got) for layer, got in loaded.items()}
