"""Engine options.  Names, meanings and defaults are those of the reference's Config
dataclass (nanovllm/config.py:6-19); the differences are listed on the fields.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, fields
from typing import Optional

from .model_config import ConfigError, canonical_dtype


@dataclass
class EngineConfig:
    model: str                              # folder with config.json and *.safetensors
    max_num_batched_tokens: int = 16384     # new tokens in one step
    max_num_seqs: int = 512                 # requests in one step
    max_model_len: int = 4096               # clamped to max_position_embeddings (config.py:25)
    gpu_memory_utilization: float = 0.9
    tensor_parallel_size: int = 1           # one GPU: only 1 is accepted
    enforce_eager: bool = False             # True: never replay a captured decode graph
    eos: int = -1                           # -1: taken from config.json / generation_config.json
    kvcache_block_size: int = 256           # any positive size (the reference demands % 256)
    num_kvcache_blocks: int = -1            # -1: sized from free device memory; a list: one count per cache group
    # beyond the reference
    dtype: Optional[str] = None             # None: config.json's; "bfloat16" or "float32"
    seed: int = 0                           # sampling seed
    schedule: str = "prefill_first"         # the reference's policy, or "mixed"
    enable_prefix_caching: bool = True
    device: str = "cuda:0"
    decode_burst: int = 16                  # decode steps in a row without the host, while no request waits (1: never)
    random_weights: Optional[int] = None    # a seed: the folder needs config.json only, weights are drawn on the device
    measure_products: bool = True           # False: product kernels for 17-256 rows by rule and record only, nothing is timed at start-up

    def __post_init__(self):
        if not os.path.isdir(self.model):                          # config.py:21
            raise ConfigError(f"model folder {self.model!r} does not exist")
        if self.tensor_parallel_size != 1:
            raise ConfigError("this engine runs on one GPU: tensor_parallel_size must be 1")
        if self.kvcache_block_size <= 0:
            raise ConfigError("kvcache_block_size must be positive")
        if self.max_num_batched_tokens <= 0 or self.max_num_seqs <= 0 or self.max_model_len <= 0:
            raise ConfigError("max_num_batched_tokens, max_num_seqs and max_model_len must be positive")
        if not (0 < self.gpu_memory_utilization <= 1):
            raise ConfigError("gpu_memory_utilization must lie in (0, 1]")
        if self.decode_burst < 1:
            raise ConfigError("decode_burst must be at least 1")
        if self.schedule not in ("prefill_first", "mixed"):
            raise ConfigError(f"schedule must be 'prefill_first' or 'mixed', got {self.schedule!r}")
        if self.dtype is not None:
            self.dtype = canonical_dtype(self.dtype)
            if self.dtype not in ("bfloat16", "float32"):
                raise ConfigError(f"dtype {self.dtype!r} has no kernels: use bfloat16 or float32")

    @classmethod
    def field_names(cls):
        return {f.name for f in fields(cls)}
