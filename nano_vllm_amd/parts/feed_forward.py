"""Feed-forward parts.

"swiglu": m = (silu(y Wg^T) * (y Wu^T)) Wd^T with gate and up packed into one matrix
[2*inner, hidden], gate rows first (nanovllm/models/qwen3.py:91-117, linear.py:87-93,
activation.py:8-11).  Dense: no experts, no routing.
"""
from __future__ import annotations

from typing import Dict, Mapping

from .base import BuildContext, ParamDecl, Part, Source
from .registry import register_part


class SwiGLU(Part):
    """params: hidden_size, intermediate_size; optional names of the checkpoint tensors."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        self.hidden = int(params["hidden_size"])
        self.inner = int(params["intermediate_size"])
        self.gate_name = params.get("gate_name", "gate_proj")
        self.up_name = params.get("up_name", "up_proj")
        self.down_name = params.get("down_name", "down_proj")

    def param_decls(self) -> Dict[str, ParamDecl]:
        i, h = self.inner, self.hidden
        return {
            "gate_up_proj.weight": ParamDecl((2 * i, h), sources=(
                Source(f"{self.gate_name}.weight", 0, i), Source(f"{self.up_name}.weight", i, i))),
            f"{self.down_name}.weight": ParamDecl((h, i)),
        }

    def forward(self, x, batch=None):
        z = self.kernels.linear_silu_mul(x, self.weights["gate_up_proj.weight"])
        # deferred: the block hands this to the next norm only
        return self.kernels.linear(z, self.weights[f"{self.down_name}.weight"], deferred=True)


register_part("feed_forward", "swiglu", SwiGLU)
