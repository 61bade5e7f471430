"""Position encodings.

A position encoding part offers two things to a mixer:
  rotary_table()   a float32 table [positions, head_dim] (cosines, then sines) when the
                   encoding is a rotation of the pairs (i, i + head_dim/2), which the mixer's
                   fused kernel applies itself; None otherwise
  apply(q, k, positions, num_heads, num_kv_heads, head_dim)
                   encodes q [T, heads*head_dim] and k [T, kv_heads*head_dim] in place; the
                   mixer calls it when there is no table

"rotary_neox": nanovllm/layers/rotary_embedding.py:17-48 - inv_freq_i = 1 / theta^(2i/D) and
angle = position * inv_freq_i in float32 whatever the model's element type, pairs (i, i+D/2).
"none": no encoding.
"""
from __future__ import annotations

from typing import Mapping, Optional

import torch

from .base import BuildContext, Part
from .registry import register_part


class RotaryNeox(Part):
    """params: head_dim, theta, max_position (rows of the table)."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        self.head_dim = int(params["head_dim"])
        self.theta = float(params["theta"])
        self.max_position = int(params.get("max_position", build.max_position))
        if self.head_dim % 2:
            raise ValueError(f"rotary_neox: head_dim {self.head_dim} must be even")
        # The reference's own float32 expression (rotary_embedding.py:29), evaluated on the host:
        # the angles' rounding is part of the model.
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, self.head_dim, 2, dtype=torch.float) / self.head_dim))
        self.inv_freq = inv_freq
        self._device = build.device
        self._table = None

    def rotary_table(self) -> Optional[torch.Tensor]:
        if self._table is None:            # made on first use: building a part touches no device
            self._table = self.kernels.rotary_table(self.inv_freq.to(self._device), self.max_position)
        return self._table

    def apply(self, q, k, positions, num_heads, num_kv_heads, head_dim):
        raise NotImplementedError("rotary_neox is applied through its table")


class NoPositionEncoding(Part):
    def rotary_table(self):
        return None

    def apply(self, q, k, positions, num_heads, num_kv_heads, head_dim):
        return None


register_part("position_encoding", "rotary_neox", RotaryNeox)
register_part("position_encoding", "none", NoPositionEncoding)
