"""The model: parts put together as a ModelSpec says.

Reference for the whole: nanovllm/models/qwen3.py:162-216 (embedding, the layers in order,
final norm, output head with optionally tied embedding).  Here the layers and their order
are data, and embedding and head are parts chosen by kind like the others (a scaled embedding
or a head with a cap on its logits is another kind, registered): Model knows no architecture.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from .base import BuildContext, ParamDecl, Part, named_params
from .registry import make_part
from .spec import LayerRun, ModelSpec, PartSpec

_TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def torch_dtype(name: str) -> torch.dtype:
    try:
        return _TORCH_DTYPES[name]
    except KeyError:
        raise ValueError(f"element type {name!r} has no kernels: use bfloat16 or float32") from None


@dataclass
class LayerCache:
    """What one run of the order owns in the cache: the index of its page group in the
    step's batch and its tensors there, or its per-request state tensors [slots, ...]."""
    group: int = -1
    k: Optional[torch.Tensor] = None
    v: Optional[torch.Tensor] = None
    state: Optional[Dict[str, torch.Tensor]] = None


class Model:
    def __init__(self, spec: ModelSpec, kernels, device="cuda:0", dtype: Optional[torch.dtype] = None):
        spec.validate()
        self.spec = spec
        self.kernels = kernels
        self.device = torch.device(device)
        self.dtype = dtype or torch_dtype(spec.dtype)
        build = BuildContext(kernels, self.device, self.dtype, spec.hidden_size, spec.max_position)
        for name, pe in spec.position_encodings.items():
            build.position_encodings[name] = make_part("position_encoding", pe, build)
        self.position_encodings = build.position_encodings
        sizes = {"vocab_size": spec.vocab_size, "hidden_size": spec.hidden_size}
        self.embedding = make_part("embedding", PartSpec(spec.embedding.kind, {**spec.embedding.params, **sizes}), build)
        self.blocks: List[Part] = []
        for layer in spec.layers:
            block_spec = PartSpec(layer.block.kind, {**layer.block.params, "parts": layer.parts, "names": layer.names})
            self.blocks.append(make_part("block", block_spec, build))
        self.final_norm = make_part("norm", spec.final_norm, build)
        self.head = make_part("head", PartSpec(spec.head.kind, {**spec.head.params, **sizes}), build)
        self.order: Tuple[LayerRun, ...] = spec.order

        # full parameter name -> (owner part, local name, declaration)
        self.param_table: Dict[str, Tuple[Part, str, ParamDecl]] = {}
        roots = [(spec.embedding["name"], self.embedding), (spec.final_norm["name"], self.final_norm),
                 (spec.head["name"], self.head)]
        roots += [(layer.name, block) for layer, block in zip(spec.layers, self.blocks)]
        for prefix, part in roots:
            for full, owner, local, decl in named_params(part, prefix):
                if full in self.param_table:
                    raise ValueError(f"two parts declare the parameter {full!r}")
                self.param_table[full] = (owner, local, decl)
        self.params: Dict[str, torch.Tensor] = {}

    # ------------------------------------------------------------------ weights
    def set_param(self, name: str, tensor: torch.Tensor) -> None:
        owner, local, decl = self.param_table[name]
        if tuple(tensor.shape) != tuple(decl.shape):
            raise ValueError(f"parameter {name}: shape {tuple(tensor.shape)} is not {tuple(decl.shape)}")
        self.params[name] = tensor
        owner.weights[local] = tensor

    def finish_weights(self) -> None:
        missing = [n for n in self.param_table if n not in self.params]
        if missing:
            raise ValueError(f"parameters without a tensor: {missing}")
        if getattr(self.head, "tied", False):
            self.head.weights["weight"] = self.embedding.weights["weight"]

        def told(part: Part) -> None:
            for child in part.children().values():
                told(child)
            part.on_weights_loaded()
        for part in [*self.position_encodings.values(), self.embedding, *self.blocks, self.final_norm, self.head]:
            told(part)

    def num_parameters(self) -> int:
        return sum(int(torch.tensor(d.shape).prod()) for _, _, d in self.param_table.values())

    # ------------------------------------------------------------------ cache
    def cache_needs(self):
        """Per entry of the order: what its cache must hold, or None when it reads another's."""
        return [self.blocks[run.layer].cache_need() if run.cache_of is None else None for run in self.order]

    def cache_owner(self, i: int) -> int:
        run = self.order[i]
        return i if run.cache_of is None else run.cache_of

    # ------------------------------------------------------------------ forward
    def forward(self, batch, caches: List[LayerCache]) -> torch.Tensor:
        """Hidden states [T, hidden] of the batch's tokens after the final norm."""
        batch.step_cache = {}        # what kernels share between the layers of one pass (a plan made by the first)
        h = self.embedding.forward(batch.input_ids)
        residual = None
        for i, run in enumerate(self.order):
            h, residual = self.blocks[run.layer].forward(h, residual, batch, caches[self.cache_owner(i)])
        if residual is None:
            return self.final_norm.forward(h)
        h, _ = self.final_norm.forward_add(h, residual)
        return h

    def logits(self, hidden: torch.Tensor, rows: Optional[torch.Tensor]) -> torch.Tensor:
        """float32 [R, vocab] at the given flat token indices (all tokens if None)."""
        x = hidden if rows is None else self.kernels.gather_rows(hidden, rows)
        return self.head.forward(x)
