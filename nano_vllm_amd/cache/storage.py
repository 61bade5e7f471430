"""Device tensors of the cache: for every run of the model's order that keeps keys and
values, K [pages, kv_heads, page, head_dim] and V [pages, kv_heads, page / vt, head_dim, vt]
of its group's page count; for every run with fixed state, its tensors [slots + 1, ...] (the
last row belongs to no request: rows that pad a captured batch read and write it).

Reference: nanovllm/engine/model_runner.py:103-121 keeps one tensor [2, layers, pages,
page, kv_heads, head_dim].  Here a (page, kv head) block is contiguous, and V is stored
transposed, in tiles of vt keys, so that the keys of one channel are contiguous for the
attention kernels (kernels.ops.v_cache_shape).
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from ..kernels.ops import v_cache_shape
from ..parts.model import LayerCache, torch_dtype


def bytes_per_page(needs, groups, page_size: int, itemsize: int) -> List[int]:
    """Per group: bytes that one page takes over all the group's runs."""
    return [sum(2 * needs[r].num_kv_heads * needs[r].head_dim * page_size * itemsize for r in g.runs)
            for g in groups]


def state_bytes_per_slot(needs, state_runs) -> int:
    total = 0
    for r in state_runs:
        for shape, dtype in needs[r].tensors.values():
            n = 1
            for s in shape:
                n *= s
            total += n * torch.empty((), dtype=_state_dtype(dtype)).element_size()
    return total


def _state_dtype(name: str) -> torch.dtype:
    return torch.float32 if name == "float32" else torch_dtype(name)


def allocate(needs, groups, state_runs, num_pages: Sequence[int], page_size: int, num_slots: int,
             dtype: torch.dtype, device) -> List[LayerCache]:
    caches: List[LayerCache] = [LayerCache() for _ in needs]
    for g, group in enumerate(groups):
        for r in group.runs:
            need = needs[r]
            k = torch.zeros((num_pages[g], need.num_kv_heads, page_size, need.head_dim), dtype=dtype, device=device)
            v = torch.zeros(v_cache_shape(num_pages[g], need.num_kv_heads, need.head_dim, page_size), dtype=dtype,
                            device=device)
            caches[r] = LayerCache(group=g, k=k, v=v)
    for r in state_runs:
        caches[r] = LayerCache(state={
            # one row more than requests can hold: the slot of the rows that pad a captured batch
            name: torch.zeros((num_slots + 1,) + tuple(shape), dtype=_state_dtype(dt), device=device)
            for name, (shape, dt) in needs[r].tensors.items()})
    return caches
