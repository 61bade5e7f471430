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
The reference rotates the whole head (qwen3.py:49-54 passes rotary_dim = head_dim); with a
smaller rotary_dim R the table is R wide and the first R channels of a head are rotated, in
pairs (i, i + R/2), the others left as they are.
"none": no encoding.
"""
from __future__ import annotations

from typing import Mapping, Optional

import torch

from .base import BuildContext, Part
from .registry import register_part


class RotaryNeox(Part):
    """params: head_dim, theta, max_position (rows of the table), rotary_dim (channels of a head
    that are rotated; default all)."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        self.head_dim = int(params["head_dim"])
        self.theta = float(params["theta"])
        self.max_position = int(params.get("max_position", build.max_position))
        rotary_dim = params.get("rotary_dim")
        self.rotary_dim = self.head_dim if rotary_dim is None else int(rotary_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_neox: {self.rotary_dim} rotated channels of a head of {self.head_dim}: "
                             f"the number must be even and at most the head's")
        # The reference's own float32 expression (rotary_embedding.py:29), evaluated on the host:
        # the angles' rounding is part of the model.
        inv_freq = 1.0 / (self.theta ** (torch.arange(0, self.rotary_dim, 2, dtype=torch.float) / self.rotary_dim))
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
