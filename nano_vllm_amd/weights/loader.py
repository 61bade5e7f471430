"""Fills a model's parameters from the safetensors files of a folder, by tensor name.

Reference: nanovllm/utils/loader.py:12-28 and the weight_loader hooks of
nanovllm/layers/linear.py:87-128 - every tensor of every *.safetensors file is copied into
the parameter (or the row range of a packed parameter) that its name selects, cast to the
parameter's type.  Unlike the reference, nothing is left unnoticed: one WeightError lists
the tensors that are missing, unexpected or of the wrong shape.

Element types: a parameter of type "model" takes the model's element type; "stored32"
(small vectors such as norm weights) stays float32 if the file stores float32; integer
tensors are kept as int32.
"""
from __future__ import annotations

import glob
import os
from dataclasses import dataclass
from typing import Dict, Tuple

import torch
from safetensors import safe_open


class WeightError(ValueError):
    def __init__(self, missing=(), unexpected=(), wrong_shape=(), other=()):
        self.missing, self.unexpected = list(missing), list(unexpected)
        self.wrong_shape, self.other = list(wrong_shape), list(other)
        lines = ["the checkpoint does not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n} is {list(got)}, expected {list(want)}" for n, got, want in self.wrong_shape))
        for o in self.other:
            lines.append("  " + o)
        super().__init__("\n".join(lines))


@dataclass(frozen=True)
class Slot:
    """Where a checkpoint tensor lands: rows [row, row+rows) of a parameter (the whole of it
    when the parameter has a single source)."""
    param: str
    row: int
    rows: int
    shape: Tuple[int, ...]       # the checkpoint tensor's expected shape
    whole: bool


def checkpoint_layout(model) -> Dict[str, Slot]:
    """checkpoint tensor name -> Slot, from the parameters the model's parts declare."""
    layout: Dict[str, Slot] = {}
    for full, (_, local, decl) in model.param_table.items():
        prefix = full[: len(full) - len(local)]          # ends with "."
        if decl.sources is None:
            layout[full] = Slot(full, 0, decl.shape[0] if decl.shape else 1, tuple(decl.shape), True)
        else:
            for src in decl.sources:
                name = prefix + src.name
                if name in layout:
                    raise ValueError(f"two parameters claim the checkpoint tensor {name!r}")
                layout[name] = Slot(full, src.row, src.rows, (src.rows,) + tuple(decl.shape[1:]), False)
    return layout


def _param_dtype(decl, stored: torch.dtype, model_dtype: torch.dtype) -> torch.dtype:
    if decl.dtype == "model":
        return model_dtype
    if decl.dtype == "stored32":
        return torch.float32 if stored == torch.float32 else model_dtype
    if decl.dtype == "float32":
        return torch.float32
    if decl.dtype == "int32":
        return torch.int32
    raise ValueError(f"unknown parameter type {decl.dtype!r}")


def load_weights(model, folder: str) -> None:
    files = sorted(glob.glob(os.path.join(folder, "*.safetensors")))
    if not files:
        raise WeightError(other=[f"{folder!r} holds no *.safetensors file"])
    layout = checkpoint_layout(model)
    tied_head = model.spec.head["name"] + ".weight" if getattr(model.head, "tied", False) else None
    seen, unexpected, wrong = set(), [], []
    tensors: Dict[str, torch.Tensor] = {}
    tied_copy = None
    for path in files:
        with safe_open(path, "pt", "cpu") as f:
            for name in f.keys():
                if name == tied_head:
                    tied_copy = f.get_tensor(name)       # checked against the embedding below
                    continue
                slot = layout.get(name)
                if slot is None:
                    unexpected.append(name)
                    continue
                if name in seen:
                    unexpected.append(f"{name} (stored twice)")
                    continue
                seen.add(name)
                shape = tuple(f.get_slice(name).get_shape())
                if shape != slot.shape:
                    wrong.append((name, shape, slot.shape))
                    continue
                t = f.get_tensor(name)
                _, _, decl = model.param_table[slot.param]
                if slot.param not in tensors:
                    if t.dtype in (torch.int64, torch.int32, torch.int16, torch.int8, torch.uint8) and decl.dtype != "int32":
                        wrong.append((name + f" (integer {t.dtype})", shape, slot.shape))
                        continue
                    tensors[slot.param] = torch.empty(decl.shape, dtype=_param_dtype(decl, t.dtype, model.dtype),
                                                      device=model.device)
                dst = tensors[slot.param]
                dst = dst if slot.whole else dst.narrow(0, slot.row, slot.rows)
                dst.copy_(t.to(dst.dtype))
    missing = sorted(n for n in layout if n not in seen)
    if missing or unexpected or wrong:
        raise WeightError(missing, sorted(unexpected), wrong)
    for name, t in tensors.items():
        model.set_param(name, t)
    model.finish_weights()
    if tied_copy is not None:
        emb = model.embedding.weights["weight"]
        if tuple(tied_copy.shape) != tuple(emb.shape) or not torch.equal(tied_copy.to(emb.dtype).to(emb.device), emb):
            raise WeightError(other=[f"{tied_head} is stored although the embeddings are tied, and differs "
                                     "from the embedding"])
