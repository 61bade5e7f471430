"""Blocks: the arrangement of a layer's parts.

"pre_norm_residual": the pre-norm residual layer with the residual sum deferred into the
next norm (nanovllm/models/qwen3.py:146-159):
    first layer:  r = h;           x = norm1(h)
    later layers: r = h + r;       x = norm1(r)
    a = mixer(x);  r = a + r;  y = norm2(r);  m = feed_forward(y);  returns (m, r)
The caller adds the last m to r inside the final norm (qwen3.py:182).

Interface of a block: forward(h, residual | None, batch, cache) -> (h, residual).
"""
from __future__ import annotations

from typing import Dict, Mapping

from .base import BuildContext, Part
from .registry import make_part, register_part


class PreNormResidualBlock(Part):
    ROLES = ("mixer_norm", "mixer", "feed_forward_norm", "feed_forward")

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        parts = params["parts"]            # role -> PartSpec
        names = params["names"]            # role -> name in checkpoint tensor names
        missing = [r for r in self.ROLES if r not in parts]
        if missing:
            raise ValueError(f"pre_norm_residual block: missing parts {missing}")
        self.mixer_norm = make_part("norm", parts["mixer_norm"], build)
        self.mixer = make_part("mixer", parts["mixer"], build)
        self.feed_forward_norm = make_part("norm", parts["feed_forward_norm"], build)
        self.feed_forward = make_part("feed_forward", parts["feed_forward"], build)
        self._children = {names[r]: getattr(self, r) for r in self.ROLES}

    def children(self) -> Dict[str, Part]:
        return self._children

    def cache_need(self):
        return self.mixer.cache_need()

    @property
    def replays_state_steps(self):
        return self.mixer.replays_state_steps

    def forward(self, h, residual, batch, cache):
        if residual is None:
            x, residual = self.mixer_norm.forward(h), h
        else:
            x, residual = self.mixer_norm.forward_add(h, residual)
        a = self.mixer.forward(x, batch, cache)
        y, residual = self.feed_forward_norm.forward_add(a, residual)
        m = self.feed_forward.forward(y, batch)
        return m, residual


register_part("block", "pre_norm_residual", PreNormResidualBlock)
