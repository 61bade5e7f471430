"""The scheduler: admits requests, cuts prompts into portions under a token budget,
decodes, finishes and frees.  Host only (no torch).

Reference: nanovllm/engine/scheduler.py:8-92.  Policy "prefill_first" is the reference's:
while requests wait, a step holds only prompt tokens (whole prompts, and a portion of the
first one if it does not fit the budget); otherwise every running request decodes one token.
Policy "mixed" puts the running requests' single tokens and portions of waiting prompts into
the same step.

When pages run out:
  * a waiting request whose pages are not free stays at the head of the queue until running
    requests end (scheduler.py:37-38);
  * a running request that needs a page for its next token takes it from the request that
    was admitted last: that one is preempted - its pages are given back, it returns to the
    front of the waiting queue and is computed again from its tokens, prompt and generated
    (scheduler.py:60-65,75-79); under "mixed" the request admitted last may still be at the
    head of the waiting queue with a part of its prompt in the cache, and is then the first
    to give its pages back;
  * a request that is alone and still cannot grow is finished with reason "cache_full"
    (the reference asserts, scheduler.py:71); a prompt that can never fit the pool is
    refused when it is added.
"""
from __future__ import annotations

from collections import deque
from typing import Deque, Iterable, List, Sequence as Seq, Tuple

from ..cache.manager import CacheManager
from .sequence import Sequence, SequenceStatus


class Scheduler:
    def __init__(self, cache: CacheManager, max_num_seqs: int, max_num_batched_tokens: int, max_model_len: int,
                 eos: Iterable[int] = (), policy: str = "prefill_first"):
        if policy not in ("prefill_first", "mixed"):
            raise ValueError(f"unknown policy {policy!r}")
        self.cache = cache
        self.page_size = cache.page_size
        self.max_num_seqs = max_num_seqs
        self.max_num_batched_tokens = max_num_batched_tokens
        self.max_model_len = max_model_len
        self.eos = set(int(e) for e in eos if e is not None and int(e) >= 0)
        self.policy = policy
        self.waiting: Deque[Sequence] = deque()
        self.running: Deque[Sequence] = deque()
        self.num_preemptions = 0
        self.just_finished: List[Sequence] = []     # finished since the engine last looked

    # ------------------------------------------------------------------ queue
    def is_finished(self) -> bool:
        return not self.waiting and not self.running

    def add(self, seq: Sequence) -> None:
        if seq.num_tokens >= self.max_model_len:
            raise ValueError(f"a prompt of {seq.num_tokens} tokens leaves no room below max_model_len "
                             f"{self.max_model_len}")
        # the prompt and one more token, group by group: a window group never holds the whole prompt
        need = self.cache.peak_pages(seq.num_tokens + 1, self.max_num_batched_tokens)
        # A window group's need is known to the end: while the request decodes it holds the pages of
        # one window, wherever that lies, however short the prompt was.  (The all-keys group grows
        # with every token; what happens when it runs out is the scheduler's business, see above.)
        final = min(seq.num_tokens + seq.max_tokens, self.max_model_len)
        for g, pages in enumerate(self.cache.peak_pages(final, 1)):
            if self.cache.groups[g].window is not None:
                need[g] = max(need[g], pages)
        for g, (pages, pool) in enumerate(zip(need, self.cache.pools)):
            if pages > pool.num_pages:
                raise ValueError(f"a prompt of {seq.num_tokens} tokens with up to {seq.max_tokens} more needs {pages} "
                                 f"pages of cache group {g}; it has {pool.num_pages}")
        self.waiting.append(seq)

    # ------------------------------------------------------------------ one step's decision
    def schedule(self) -> Tuple[List[Sequence], bool]:
        """The requests of the next step, each with num_scheduled_tokens set and its pages
        reserved, and whether the step holds prompt tokens only (the reference's is_prefill)."""
        if self.policy == "mixed":
            return self._schedule_mixed()
        batch, budget = self._schedule_prompts([], self.max_num_batched_tokens)
        if batch:
            return batch, True
        batch = self._schedule_decodes()
        return batch, False

    def _schedule_prompts(self, batch: List[Sequence], budget: int):
        """scheduler.py:29-52."""
        first_here = len(batch)
        while self.waiting and len(batch) < self.max_num_seqs and budget > 0:
            seq = self.waiting[0]
            if not seq.admitted:
                # all keys: every page of the prompt at admission, as the reference does; a window
                # group takes the pages of each portion when its step comes
                hits = self.cache.can_admit(seq.token_ids, budget)
                if hits == -1:
                    break
                todo = seq.num_tokens - hits * self.page_size
            else:
                todo = seq.num_tokens - seq.num_cached_tokens
            if budget < todo and len(batch) > first_here:       # only the first prompt of a step is cut
                break
            if not seq.admitted:
                seq.num_cached_tokens = self.cache.admit_with_prefix(seq.seq_id, seq.token_ids, budget)
                seq.admitted = True
            else:
                end = seq.num_cached_tokens + min(todo, budget)
                if not self.cache.can_reserve(seq.seq_id, seq.num_tokens, seq.num_cached_tokens, step_end=end):
                    break                                       # a window group waits for pages of running requests
                self.cache.reserve(seq.seq_id, seq.num_tokens, seq.num_cached_tokens, step_end=end)
            seq.num_scheduled_tokens = min(todo, budget)
            budget -= seq.num_scheduled_tokens
            if seq.num_cached_tokens + seq.num_scheduled_tokens == seq.num_tokens:
                seq.status = SequenceStatus.RUNNING
                self.waiting.popleft()
                self.running.append(seq)
            batch.append(seq)
        return batch, budget

    def _schedule_decodes(self) -> List[Sequence]:
        """scheduler.py:57-73."""
        batch: List[Sequence] = []
        while self.running and len(batch) < self.max_num_seqs:
            seq = self.running.popleft()
            while not self.cache.can_reserve(seq.seq_id, seq.num_tokens, first_query=seq.num_tokens - 1):
                if self.waiting and self.waiting[0].admitted:
                    # policy "mixed": the request admitted last is still being cut into portions and
                    # holds pages at the head of the waiting queue; it is the newest, so it goes first
                    self._preempt_waiting_head()
                elif self.running:
                    self.preempt(self.running.pop())
                elif batch:
                    self.preempt(seq)
                    break
                else:
                    self._finish(seq, "cache_full")              # alone and cannot grow
                    break
            else:
                self.cache.reserve(seq.seq_id, seq.num_tokens, first_query=seq.num_tokens - 1)
                seq.num_scheduled_tokens = 1
                batch.append(seq)
        self.running.extendleft(reversed(batch))
        return batch

    def _schedule_mixed(self) -> Tuple[List[Sequence], bool]:
        # Requests that were running before this step decode; those whose prompt ends in this
        # step join `running` but must not decode in it as well.
        before = self.num_preemptions
        decodes = self._schedule_decodes()
        if self.num_preemptions != before:
            return decodes, False        # pages were just taken away: admit nothing in this step
        budget = self.max_num_batched_tokens - len(decodes)
        batch, _ = self._schedule_prompts(list(decodes), budget)
        return batch, len(decodes) == 0 and len(batch) > 0

    def preempt(self, seq: Sequence) -> None:
        """scheduler.py:75-79."""
        self._take_pages_away(seq)
        self.waiting.appendleft(seq)

    def _preempt_waiting_head(self) -> None:
        """The same for a request that holds pages but has not left the waiting queue yet (its
        prompt is not all in the cache): it keeps its place at the head."""
        self._take_pages_away(self.waiting[0])

    def _take_pages_away(self, seq: Sequence) -> None:
        self.num_preemptions += 1
        seq.status = SequenceStatus.WAITING
        self.cache.release(seq.seq_id)
        seq.admitted = False
        seq.num_cached_tokens = 0
        seq.num_scheduled_tokens = 0

    # ------------------------------------------------------------------ after the step
    def postprocess(self, seqs: Seq[Sequence], token_ids: Seq[int]) -> None:
        """scheduler.py:81-92.  token_ids: one per request of the step; ignored for a request
        whose known tokens are not all in the cache yet."""
        for seq, token_id in zip(seqs, token_ids):
            if seq.is_finished:
                continue
            done = seq.num_cached_tokens + seq.num_scheduled_tokens
            self.cache.register_full_pages(seq.seq_id, seq.token_ids, done)
            seq.num_cached_tokens = done
            seq.num_scheduled_tokens = 0
            if seq.num_cached_tokens < seq.num_tokens:
                continue
            seq.append_token(int(token_id))
            if not seq.ignore_eos and int(token_id) in self.eos:
                self._finish(seq, "eos")
            elif seq.num_completion_tokens >= seq.max_tokens:
                self._finish(seq, "max_tokens")
            elif seq.num_tokens >= self.max_model_len:
                self._finish(seq, "length")

    def _finish(self, seq: Sequence, reason: str) -> None:
        seq.status = SequenceStatus.FINISHED
        seq.finish_reason = reason
        self.just_finished.append(seq)
        if seq.admitted:
            self.cache.release(seq.seq_id)
            seq.admitted = False
        if seq in self.running:
            self.running.remove(seq)
