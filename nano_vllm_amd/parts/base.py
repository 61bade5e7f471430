"""What every part is: a holder of named parameters with a forward method.

A part declares its parameters (local name -> ParamDecl); the model allocates them, the
loader fills them by checkpoint tensor name, and the part reads them from self.weights.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Mapping, Optional, Tuple

import torch


@dataclass(frozen=True)
class Source:
    """A checkpoint tensor that fills rows [row, row + rows) of a parameter."""
    name: str                 # name below the part's prefix, e.g. "q_proj.weight"
    row: int
    rows: int


@dataclass(frozen=True)
class ParamDecl:
    shape: Tuple[int, ...]
    # "model": the model's element type; "stored32": float32 if the checkpoint stores float32,
    # else the model's element type; "float32"; "int32" (integer tables)
    dtype: str = "model"
    sources: Optional[Tuple[Source, ...]] = None     # None: one tensor of the parameter's own name
    init: str = "normal"                             # random-weights mode: "normal" | "norm"


@dataclass
class BuildContext:
    """What a part may use while it is built."""
    kernels: object                   # the operations (kernels.ops.HipKernels or a stand-in of the same methods)
    device: torch.device
    dtype: torch.dtype                # the model's element type
    hidden_size: int
    max_position: int
    position_encodings: Dict[str, object] = field(default_factory=dict)


class Part:
    """Base of mixers, feed-forwards, norms, position encodings and blocks."""

    # A mixer with per-request state says True when its forward, for a step of single tokens,
    # reads the step's metadata on the device only (batch.state_slots, batch.seq_starts, ... as
    # tensors; no .tolist() or .item(), nothing decided on the host from their values): such a step
    # can be captured once and replayed for other requests.  Rows that pad a captured batch carry a
    # state slot of their own that no request holds (the state tensors' last row).
    replays_state_steps = False

    def __init__(self, params: Mapping, build: BuildContext):
        self.params = dict(params)
        self.kernels = build.kernels
        self.weights: Dict[str, torch.Tensor] = {}

    def param_decls(self) -> Dict[str, ParamDecl]:
        return {}

    def children(self) -> Dict[str, "Part"]:
        """Sub-parts, by the name under which their parameters appear."""
        return {}

    def on_weights_loaded(self) -> None:
        """Called once every parameter is filled (derived tensors are made here)."""


def named_params(part: Part, prefix: str) -> List[Tuple[str, Part, str, ParamDecl]]:
    """(full parameter name, owner, local name, declaration) of a part and its sub-parts."""
    out = []
    for local, decl in part.param_decls().items():
        out.append((f"{prefix}.{local}" if prefix else local, part, local, decl))
    for name, child in part.children().items():
        out.extend(named_params(child, f"{prefix}.{name}" if prefix and name else (prefix or name)))
    return out
