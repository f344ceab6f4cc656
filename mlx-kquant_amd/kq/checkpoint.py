"""The kquant checkpoint format on disk, for torch state dicts: `config.json` + (sharded) safetensors, as
the reference's converter writes and its loader reads (docs/integration.md:73-95, mlx_kquant/convert.py:208-238,
mlx_kquant/loader.py:98-175).

  config.json       carries {"mode": "kquant", "per_tensor": {bare module path: codec}} twice, under
                    "quantization" and a mirrored "quantization_config"
  <path>.weight     uint8 [out, bytes_per_row] or [E, out, bytes_per_row]: the wire bytes
  <path>.scales     uint8 [1] placeholder (the real scales live inside the wire bytes)
  <path>.bias       optional, source dtype
  everything else   source dtype, untouched

`quantize_state` encodes float weights with kq.quantize, `save` / `load` move the result to and from disk, and
`install` swaps the named torch.nn.Linear / torch.nn.Embedding leaves of a model for the wire-byte modules
of kq.nn (the counterpart of the reference's install_kquant_modules for torch models).
"""
from __future__ import annotations

import json
import os
from typing import Dict, Mapping, NamedTuple, Optional

import torch

import kq

from . import nn as kqnn
from .codec_geometry import CODEC_GEOMETRY, in_features

_INDEX = "model.safetensors.index.json"


class Checkpoint(NamedTuple):
    config: dict
    per_tensor: Dict[str, str]          # bare module path -> codec
    tensors: Dict[str, torch.Tensor]    # every tensor of the checkpoint, by its key


def _check_quantized(path: str, codec: str, tensors: Mapping[str, torch.Tensor]):
    if codec not in CODEC_GEOMETRY:
        raise ValueError(f"{path}: unknown codec '{codec}'")
    w = tensors.get(path + ".weight")
    if w is None:
        raise ValueError(f"{path}: per_tensor names it but '{path}.weight' is missing")
    if w.dtype != torch.uint8 or w.ndim not in (2, 3):
        raise ValueError(f"{path}.weight must be uint8 [out, bytes_per_row] or [E, out, bytes_per_row]")
    in_features(codec, w.shape[-1])  # raises when the row is not a whole number of blocks


def quantize_state(state: Mapping[str, torch.Tensor], recipe: Mapping[str, str],
                   imatrix: Optional[Mapping[str, torch.Tensor]] = None):
    """Encode `<path>.weight` ([out, in] or [E, out, in], float) for every path in `recipe` (path -> codec);
    every other tensor passes through.  Returns (tensors, per_tensor) ready for `save`."""
    out = dict(state)
    for path, codec in recipe.items():
        key = path + ".weight"
        if key not in state:
            raise ValueError(f"{path}: no '{key}' in the state dict")
        im = None if imatrix is None else imatrix.get(path)
        wq, scales = kq.quantize(state[key], codec, im)
        out[key] = wq.cpu()
        out[path + ".scales"] = scales.cpu()
    return out, dict(recipe)


def save(path: str, tensors: Mapping[str, torch.Tensor], per_tensor: Mapping[str, str], config: Optional[dict] = None,
         max_shard_bytes: int = 5 << 30):
    """Write config.json and model.safetensors (or numbered shards plus their index) under `path`."""
    from safetensors.torch import save_file

    tensors = {k: v.detach().cpu().contiguous() for k, v in tensors.items()}
    for p, codec in per_tensor.items():
        _check_quantized(p, codec, tensors)
        tensors.setdefault(p + ".scales", torch.zeros(1, dtype=torch.uint8))
    os.makedirs(path, exist_ok=True)
    block = {"mode": "kquant", "per_tensor": dict(per_tensor)}
    cfg = dict(config or {})
    cfg["quantization"] = block
    cfg["quantization_config"] = dict(block)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f, indent=2, sort_keys=True)
    shards, cur, size = [], {}, 0
    for k in sorted(tensors):
        nbytes = tensors[k].numel() * tensors[k].element_size()
        if cur and size + nbytes > max_shard_bytes:
            shards.append(cur)
            cur, size = {}, 0
        cur[k] = tensors[k]
        size += nbytes
    shards.append(cur)
    if len(shards) == 1:
        save_file(shards[0], os.path.join(path, "model.safetensors"), metadata={"format": "pt"})
        return
    weight_map, total = {}, 0
    for i, shard in enumerate(shards):
        name = f"model-{i + 1:05d}-of-{len(shards):05d}.safetensors"
        save_file(shard, os.path.join(path, name), metadata={"format": "pt"})
        for k, v in shard.items():
            weight_map[k] = name
            total += v.numel() * v.element_size()
    with open(os.path.join(path, _INDEX), "w") as f:
        json.dump({"metadata": {"total_size": total}, "weight_map": weight_map}, f, indent=2, sort_keys=True)


def load(path: str, device=None) -> Checkpoint:
    """Read a checkpoint directory written by `save` (or by the reference's converter)."""
    from safetensors.torch import load_file

    with open(os.path.join(path, "config.json")) as f:
        config = json.load(f)
    block = config.get("quantization") or config.get("quantization_config")
    if not block or block.get("mode") != "kquant":
        raise ValueError(f"{path}: config.json carries no kquant quantization block")
    per_tensor = dict(block.get("per_tensor", {}))
    files = sorted(n for n in os.listdir(path) if n.startswith("model") and n.endswith(".safetensors"))
    if not files:
        raise FileNotFoundError(f"{path}: no model*.safetensors")
    tensors: Dict[str, torch.Tensor] = {}
    for name in files:
        tensors.update(load_file(os.path.join(path, name), device="cpu"))
    for p, codec in per_tensor.items():
        _check_quantized(p, codec, tensors)
    if device is not None:
        tensors = {k: v.to(device) for k, v in tensors.items()}
    return Checkpoint(config, per_tensor, tensors)


def install(model: torch.nn.Module, ckpt: Checkpoint, device=None, strict: bool = True) -> torch.nn.Module:
    """Swap the leaves of `model` named in the checkpoint's per_tensor map for wire-byte modules
    (torch.nn.Linear -> KQuantLinear, torch.nn.Embedding -> KQuantEmbedding; a 3-D weight makes a
    KQuantSwitchLinear whatever the leaf was) and load every other tensor into the model."""
    taken = set()
    for path, codec in ckpt.per_tensor.items():
        wire = ckpt.tensors[path + ".weight"]
        bias = ckpt.tensors.get(path + ".bias")
        parent_path, _, leaf = path.rpartition(".")
        parent = model.get_submodule(parent_path) if parent_path else model
        old = getattr(parent, leaf, None)
        if old is None:
            raise ValueError(f"{path}: the model has no such module")
        k = in_features(codec, wire.shape[-1])
        if wire.ndim == 3:
            new = kqnn.KQuantSwitchLinear(wire.shape[0], wire.shape[1], k, bias is not None, codec, device=device)
        elif isinstance(old, torch.nn.Embedding):
            new = kqnn.KQuantEmbedding(wire.shape[0], k, codec, device=device)
        else:
            new = kqnn.KQuantLinear(k, wire.shape[0], bias is not None, codec, device=device)
        new.load_wire(wire, bias)
        setattr(parent, leaf, new)
        taken.update({path + ".weight", path + ".scales", path + ".bias"})
    rest = {k: v for k, v in ckpt.tensors.items() if k not in taken}
    missing, unexpected = model.load_state_dict(rest, strict=False)
    missing = [k for k in missing if k not in taken]  # the swapped leaves were filled by load_wire
    if strict and (missing or unexpected):
        raise ValueError(f"install: missing {sorted(missing)}, unexpected {sorted(unexpected)}")
    if device is not None:
        model.to(device)
    return model
