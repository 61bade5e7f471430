"""Random-weights mode: makes a model folder (config.json, model.safetensors) from a
configuration and a seed, or fills a built model in place on its device.

The reference has no such mode.  Matrices are N(0, std); norm weights are 1, or
1 + N(0, norm_std) when norm_std > 0.  Checkpoint tensors are drawn in the sorted order of
their names from one seeded CPU generator, in float32, then cast: the values do not depend
on how the engine packs them.
"""
from __future__ import annotations

import json
import os
import zlib
from typing import Dict, Optional

import torch
from safetensors.torch import save_file

from ..config.registry import architecture_of
from ..parts.model import Model, torch_dtype
from .loader import checkpoint_layout


def _declaration_model(config_json: dict) -> Model:
    """The model's parts without a device: only their parameter declarations are used."""
    arch = architecture_of(config_json)
    spec = arch.build_spec(arch.parse_config(config_json))
    return Model(spec, kernels=None, device="cpu")


def random_checkpoint(config_json: dict, seed: int, std: float = 0.02, norm_std: float = 0.0,
                      dtype: Optional[str] = None) -> Dict[str, torch.Tensor]:
    """checkpoint tensor name -> tensor, for the architecture config_json names."""
    model = _declaration_model(config_json)
    out_dtype = torch_dtype(dtype) if dtype else model.dtype
    layout = checkpoint_layout(model)
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    tensors = {}
    for name in sorted(layout):
        slot = layout[name]
        _, _, decl = model.param_table[slot.param]
        if decl.dtype == "int32":
            t = torch.randint(0, 2 ** 15, slot.shape, generator=gen, dtype=torch.int32)
        elif decl.init == "norm":
            t = torch.ones(slot.shape, dtype=torch.float32)
            if norm_std > 0:
                t = t + norm_std * torch.randn(slot.shape, generator=gen, dtype=torch.float32)
            t = t.to(out_dtype)
        else:
            t = (std * torch.randn(slot.shape, generator=gen, dtype=torch.float32)).to(out_dtype)
        tensors[name] = t.contiguous()
    return tensors


def write_random_model(folder: str, config, seed: int, std: float = 0.02, norm_std: float = 0.0,
                       dtype: Optional[str] = None) -> str:
    """Writes config.json and model.safetensors.  `config` is a typed configuration (with
    to_dict()) or a config.json dictionary.  dtype overrides the stored element type."""
    config_json = dict(config.to_dict() if hasattr(config, "to_dict") else config)
    if dtype:
        config_json["torch_dtype"] = dtype
        config_json.pop("dtype", None)
    os.makedirs(folder, exist_ok=True)
    tensors = random_checkpoint(config_json, seed, std, norm_std, dtype)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config_json, f, indent=2)
    save_file(tensors, os.path.join(folder, "model.safetensors"), metadata={"format": "pt"})
    return folder


def fill_random_(model: Model, seed: int, std: float = 0.02, norm_std: float = 0.0) -> None:
    """Fills a built model on its own device, one generator per parameter (seeded from the
    seed and the parameter's name): for sizes at which a CPU generator would take minutes."""
    for name, (_, _, decl) in model.param_table.items():
        gen = torch.Generator(device=model.device)
        gen.manual_seed((seed * 1000003 + zlib.crc32(name.encode())) % (2 ** 63))
        dtype = torch.int32 if decl.dtype == "int32" else (torch.float32 if decl.dtype == "float32" else model.dtype)
        if decl.dtype == "int32":
            t = torch.randint(0, 2 ** 15, decl.shape, generator=gen, dtype=torch.int32, device=model.device)
        elif decl.init == "norm":
            t = torch.ones(decl.shape, dtype=torch.float32, device=model.device)
            if norm_std > 0:
                t += norm_std * torch.randn(decl.shape, generator=gen, dtype=torch.float32, device=model.device)
            t = t.to(dtype)
        else:
            t = torch.empty(decl.shape, dtype=dtype, device=model.device)
            t.normal_(0.0, std, generator=gen)
        model.set_param(name, t)
    model.finish_weights()
