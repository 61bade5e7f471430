"""Norm parts.

"rms_norm": y = cast(x * rsqrt(mean(x^2) + eps)) * weight, and the same fused with the
residual sum (nanovllm/layers/layernorm.py:16-40).  Sizes and eps are parameters.
"""
from __future__ import annotations

from typing import Dict, Mapping

from .base import BuildContext, ParamDecl, Part
from .registry import register_part


class RMSNorm(Part):
    """params: dim, eps."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        self.dim = int(params["dim"])
        self.eps = float(params["eps"])

    def param_decls(self) -> Dict[str, ParamDecl]:
        # vectors stay in float32 when the checkpoint stores them so
        return {"weight": ParamDecl((self.dim,), dtype="stored32", init="norm")}

    def forward(self, x, out=None):
        return self.kernels.rms_norm(x, self.weights["weight"], self.eps, out=out)

    def forward_add(self, x, residual, out=None):
        """residual <- x + residual; returns (norm(residual), residual)."""
        return self.kernels.add_rms_norm(x, residual, self.weights["weight"], self.eps, out=out)


register_part("norm", "rms_norm", RMSNorm)
