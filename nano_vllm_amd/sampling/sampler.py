"""Chooses next tokens from float32 logits: argmax for temperature 0, else a draw from
softmax(logits / temperature) (nanovllm/layers/sampler.py:8-12) with noise that is a pure
function of (seed, request, position), so that a request's tokens do not depend on its
batch-mates.
"""
from __future__ import annotations

from typing import List, Sequence

import numpy as np
import torch

_M64 = (1 << 64) - 1


def _mix64(z: int) -> int:
    z = (z + 0x9E3779B97F4A7C15) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def noise_key(seed: int, request: int, position: int) -> int:
    """The 64-bit key of one draw, as a signed integer (for an int64 tensor)."""
    key = _mix64(_mix64(_mix64(seed & _M64) ^ (request & _M64)) ^ (position & _M64))
    return key - (1 << 64) if key >= (1 << 63) else key


def noise_keys(seeds: Sequence[int], requests: Sequence[int], positions: Sequence[int]) -> "np.ndarray":
    """noise_key of many draws at once, as int64 (the same integers, computed modulo 2^64)."""
    def mix(z):
        z = z + np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))

    as_u64 = lambda values: np.array([v & _M64 for v in values], dtype=np.uint64)
    with np.errstate(over="ignore"):
        return mix(mix(mix(as_u64(seeds)) ^ as_u64(requests)) ^ as_u64(positions)).view(np.int64)


class Sampler:
    """Holds the device copies of what rarely changes from step to step (the temperatures of
    the batch; the unused keys of a batch that is all greedy), so that a decode step of the
    same requests uploads nothing, or only its keys."""

    def __init__(self, kernels, device):
        self.kernels = kernels
        self.device = device
        self._temps = None            # (tuple of temperatures, device tensor)
        self._zero_keys = None

    def device_inputs(self, temperatures: Sequence[float], seeds: Sequence[int], requests: Sequence[int],
                      positions: Sequence[Sequence[int]]):
        """(temperatures float32 [n], keys int64 [len(positions), n]) on the device, for draws
        at each of the given rows of positions."""
        n = len(temperatures)
        temps = tuple(float(t) for t in temperatures)
        assert len(seeds) == n and len(requests) == n and all(len(p) == n for p in positions)
        if self._temps is None or self._temps[0] != temps:
            self._temps = (temps, torch.tensor(temps, dtype=torch.float32).to(self.device))
        rows = len(positions)
        if any(t > 0.0 for t in temps):
            keys = np.stack([noise_keys(seeds, requests, p) for p in positions])
            keys_t = torch.from_numpy(keys).to(self.device)
        else:
            if self._zero_keys is None or self._zero_keys.numel() < rows * n:
                self._zero_keys = torch.zeros(max(rows * n, 64), dtype=torch.int64, device=self.device)
            keys_t = self._zero_keys[:rows * n].view(rows, n)
        return self._temps[1], keys_t

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], seeds: Sequence[int],
               requests: Sequence[int], positions: Sequence[int]) -> List[int]:
        """One token per row of logits.  positions: the position the new token will take."""
        assert logits.shape[0] == len(temperatures)
        temps, keys = self.device_inputs(temperatures, seeds, requests, [positions])
        return self.kernels.sample(logits, temps, keys[0]).tolist()
