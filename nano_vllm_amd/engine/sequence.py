"""A request's state on the host.

Reference: nanovllm/engine/sequence.py:8-83.  The block table is not kept here but in the
cache manager, under the request's id.
"""
from __future__ import annotations

from enum import Enum, auto
from itertools import count
from typing import List, Optional

from ..sampling.params import SamplingParams


class SequenceStatus(Enum):
    WAITING = auto()
    RUNNING = auto()
    FINISHED = auto()


class Sequence:
    _ids = count()

    def __init__(self, token_ids: List[int], sampling_params: Optional[SamplingParams] = None,
                 seq_id: Optional[int] = None):
        if not token_ids:
            raise ValueError("a request needs at least one prompt token")
        sp = sampling_params or SamplingParams()
        # The reference numbers requests with one counter per process (sequence.py:16,19); an
        # engine numbers its own from 0, so that equal runs draw equal sampling noise.
        self.seq_id = next(Sequence._ids) if seq_id is None else seq_id
        self.status = SequenceStatus.WAITING
        self.token_ids = list(token_ids)
        self.num_prompt_tokens = len(token_ids)
        self.num_cached_tokens = 0        # tokens whose keys are in the cache: prefix hits and progress
        self.num_scheduled_tokens = 0     # this step's
        self.admitted = False             # holds pages in the cache manager
        self.temperature = sp.temperature
        self.max_tokens = sp.max_tokens
        self.ignore_eos = sp.ignore_eos
        self.seed = sp.seed
        self.finish_reason: Optional[str] = None

    def __len__(self):
        return len(self.token_ids)

    @property
    def num_tokens(self) -> int:
        return len(self.token_ids)

    @property
    def last_token(self) -> int:
        return self.token_ids[-1]

    @property
    def is_finished(self) -> bool:
        return self.status == SequenceStatus.FINISHED

    @property
    def num_completion_tokens(self) -> int:
        return len(self.token_ids) - self.num_prompt_tokens

    @property
    def prompt_token_ids(self) -> List[int]:
        return self.token_ids[: self.num_prompt_tokens]

    @property
    def completion_token_ids(self) -> List[int]:
        return self.token_ids[self.num_prompt_tokens:]

    def append_token(self, token_id: int) -> None:
        self.token_ids.append(token_id)
