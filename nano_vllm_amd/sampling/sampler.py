"""Chooses next tokens from float32 logits: argmax for temperature 0, else a draw from
softmax(logits / temperature) (nanovllm/layers/sampler.py:8-12) with noise that is a pure
function of (seed, request, position), so that a request's tokens do not depend on its
batch-mates.
"""
from __future__ import annotations

from typing import List, Sequence

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


class Sampler:
    def __init__(self, kernels, device):
        self.kernels = kernels
        self.device = device

    def sample(self, logits: torch.Tensor, temperatures: Sequence[float], seeds: Sequence[int],
               requests: Sequence[int], positions: Sequence[int]) -> List[int]:
        """One token per row of logits.  positions: the position the new token will take."""
        n = logits.shape[0]
        keys = [noise_key(s, r, p) for s, r, p in zip(seeds, requests, positions)]
        temps = torch.tensor(list(temperatures), dtype=torch.float32).to(self.device)
        keys_t = torch.tensor(keys, dtype=torch.int64).to(self.device)
        assert temps.shape[0] == n and keys_t.shape[0] == n
        ids = self.kernels.sample(logits, temps, keys_t)
        return ids.tolist()
