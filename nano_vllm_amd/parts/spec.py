"""A model as data: which parts make up each layer, with their sizes and constants, and
the order in which layers run.

An architecture's definition (models/*.py) turns its typed configuration into a ModelSpec;
parts.model.Model builds the parts a ModelSpec names from the part registries.  Nothing in
a part names the model it is in.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part: its kind (a name in the registry of its role) and its parameters."""
    kind: str
    params: Mapping[str, Any] = field(default_factory=dict)

    def get(self, key, default=None):
        return self.params.get(key, default)

    def __getitem__(self, key):
        return self.params[key]


@dataclass(frozen=True)
class LayerSpec:
    """One layer with weights of its own.

    block     how the parts below are arranged (a kind in the block registry)
    parts     role -> PartSpec; the roles a block knows ("mixer", "feed_forward",
              "mixer_norm", "feed_forward_norm" for the pre-norm residual block)
    name      the layer's prefix in checkpoint tensor names ("model.layers.3")
    names     role -> the part's name below that prefix ("self_attn", "mlp", ...)
    """
    block: PartSpec
    parts: Mapping[str, PartSpec]
    name: str
    names: Mapping[str, str]


@dataclass(frozen=True)
class LayerRun:
    """One entry of the execution order.

    layer     index into ModelSpec.layers: whose weights run.  A layer may be named twice.
    cache_of  None: the run has a cache of its own.  An index of an earlier entry of the
              order: the run reads that entry's cache and writes none.
    """
    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_position: int
    dtype: str                                   # "bfloat16" | "float32": config.json's
    embedding: PartSpec                          # params: name
    layers: Tuple[LayerSpec, ...]
    order: Tuple[LayerRun, ...]
    final_norm: PartSpec                         # params: name + the norm's own
    head: PartSpec                               # params: name, tied
    position_encodings: Mapping[str, PartSpec]   # shared by name among the mixers
    eos_token_ids: Tuple[int, ...] = ()

    def validate(self) -> None:
        for i, run in enumerate(self.order):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"order[{i}] names layer {run.layer}; there are {len(self.layers)}")
            if run.cache_of is not None:
                if not 0 <= run.cache_of < i:
                    raise ValueError(f"order[{i}] reads the cache of entry {run.cache_of}, which must run earlier")
                if self.order[run.cache_of].cache_of is not None:
                    raise ValueError(f"order[{i}] reads the cache of entry {run.cache_of}, which has none of its own")


# ---------------------------------------------------------------------------- cache needs
@dataclass(frozen=True)
class PagedKV:
    """Keys and values of every token, in pages.  window None: all keys stay; an integer:
    a query at position p reads positions > p - window only, and pages wholly before that
    are given back."""
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class FixedState:
    """State of fixed size per request, kept in a slot: name -> (shape, dtype name)."""
    tensors: Mapping[str, Tuple[Tuple[int, ...], str]]
