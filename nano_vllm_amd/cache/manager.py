"""The cache manager: pages and block tables for every request and cache group, and a slot
for each request's fixed-size state.  Host side only (no torch).

Layers whose caches have the same needs form a group with pages of its own: all layers that
keep every key are one group, layers with a window of w keys another.  A request has one
block table per group: entry i is the page that holds positions [i*page, (i+1)*page), or -1
where the window has passed and the page was given back.  Pages are given back when a
request is released and when a window has passed them, and are taken again from the head of
the free list.

Reference: nanovllm/engine/block_manager.py:26-120 (one group, all keys, prefix hashes).
The prefix-hash reuse of the reference works over every group: a full page is registered under
the chained hash of its tokens in each group's pool, and a new request leaves out as many leading
pages as every group can still stand for (an all-keys group all of them, a window group those the
first computed token looks at).  Where per-request state of fixed size exists, pages do not carry
all a request needs, and hits are switched off.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np
import xxhash

from .pages import OutOfPages, PageError, PagePool, SlotPool


@dataclass(frozen=True)
class CacheGroup:
    window: Optional[int]          # None: all keys
    runs: Tuple[int, ...]          # entries of the model's order that keep their cache here


@dataclass
class RequestCache:
    tables: List[List[int]]        # per group
    num_tokens: int = 0            # positions reserved so far
    state_slot: int = -1
    # chain of prefix hashes of the full pages registered so far (the same chain in every group)
    hashes: List[int] = field(default_factory=list)


def plan_groups(needs) -> Tuple[List[CacheGroup], List[int]]:
    """From the per-run needs (PagedKV / FixedState / None) the page groups, and the runs
    that keep fixed state.  A need is recognised by its attributes, so that this module
    imports nothing from the parts."""
    by_window: Dict[Optional[int], List[int]] = {}
    state_runs: List[int] = []
    for i, need in enumerate(needs):
        if need is None:
            continue
        if hasattr(need, "tensors"):
            state_runs.append(i)
        elif hasattr(need, "num_kv_heads"):
            by_window.setdefault(need.window, []).append(i)
        else:
            raise ValueError(f"run {i}: unknown cache need {need!r}")
    keys = sorted(by_window, key=lambda w: (w is not None, w or 0))       # the all-keys group first
    return [CacheGroup(w, tuple(by_window[w])) for w in keys], state_runs


def chain_hash(tokens: Sequence[int], prefix: int = -1) -> int:
    """block_manager.py:35-41: xxh64 over the previous block's hash (8 bytes, little endian)
    and the block's token ids as 64-bit integers."""
    h = xxhash.xxh64()
    if prefix != -1:
        h.update(prefix.to_bytes(8, "little"))
    h.update(np.asarray(tokens, dtype=np.int64).tobytes())
    return h.intdigest()


class CacheManager:
    def __init__(self, groups: Sequence[CacheGroup], page_size: int, num_pages, num_state_slots: int = 0,
                 has_state: bool = False, enable_prefix_caching: bool = True):
        self.groups = list(groups)
        self.page_size = page_size
        counts = list(num_pages) if isinstance(num_pages, (list, tuple)) else [num_pages] * len(self.groups)
        if len(counts) != len(self.groups):
            raise ValueError("one page count per group is needed")
        self.pools = [PagePool(n, page_size) for n in counts]
        self.slots = SlotPool(num_state_slots)
        self.has_state = has_state
        # Keys of a prefix are the same whoever computed them; state of fixed size is not kept by
        # prefix, so a model with such state computes every prompt whole.
        self.prefix_caching = enable_prefix_caching and not has_state
        self.requests: Dict[Hashable, RequestCache] = {}

    # ------------------------------------------------------------------ requests
    def admit(self, request: Hashable) -> RequestCache:
        if request in self.requests:
            raise PageError(f"request {request!r} is admitted already")
        slot = self.slots.take() if self.slots.num_slots else -1
        rc = RequestCache(tables=[[] for _ in self.groups], state_slot=slot)
        self.requests[request] = rc
        return rc

    def release(self, request: Hashable) -> None:
        """Gives back everything the request holds.  Tables are walked from the end so that a
        request's last pages are reused before its first (block_manager.py:94-101)."""
        rc = self.requests.pop(request)
        for pool, table in zip(self.pools, rc.tables):
            for page in reversed(table):
                if page >= 0:
                    pool.give_back(page)
        if rc.state_slot >= 0:
            self.slots.give_back(rc.state_slot)

    def table(self, request: Hashable, group: int) -> List[int]:
        return self.requests[request].tables[group]

    # ------------------------------------------------------------------ pages for new tokens
    def _first_needed_page(self, group: int, first_query: int) -> int:
        w = self.groups[group].window
        if w is None:
            return 0
        return max(0, first_query - w + 1) // self.page_size

    def _wanted_pages(self, group: int, new_len: int, step_end: Optional[int]) -> int:
        """The length of the group's block table that covers positions < new_len; a window group
        covers only positions < step_end, the end of the step at hand, when that is given."""
        if step_end is not None and self.groups[group].window is not None:
            new_len = min(new_len, step_end)
        return (new_len + self.page_size - 1) // self.page_size

    def pages_needed(self, request: Hashable, new_len: int, first_query: Optional[int] = None,
                     step_end: Optional[int] = None) -> List[int]:
        """Per group: the pages that must be taken so that positions < new_len are covered,
        for a step whose first query stands at position first_query (default: the first
        position not yet reserved).  With step_end, the end of that step, a window group takes
        pages up to there only: the pages further on are taken by the steps that reach them,
        when the window has passed earlier ones."""
        rc = self.requests[request]
        first_query = rc.num_tokens if first_query is None else first_query
        out = []
        for g, table in enumerate(rc.tables):
            lo = max(len(table), self._first_needed_page(g, first_query))
            out.append(max(0, self._wanted_pages(g, new_len, step_end) - lo))
        return out

    def peak_pages(self, num_tokens: int, portion: int) -> List[int]:
        """Per group: the most pages a request of num_tokens positions holds at any time when no
        step brings more than `portion` of its tokens.  The all-keys group holds every page; a
        window group holds those of one step's tokens and of the window before the first of them."""
        total = (num_tokens + self.page_size - 1) // self.page_size
        out = []
        for group in self.groups:
            if group.window is None:
                out.append(total)
            else:
                span = group.window - 1 + max(1, min(portion, num_tokens))       # positions a step touches, at any offset
                out.append(min(total, (span + self.page_size - 2) // self.page_size + 1))
        return out

    def can_reserve(self, request: Hashable, new_len: int, first_query: Optional[int] = None,
                    step_end: Optional[int] = None) -> bool:
        need = self.pages_needed(request, new_len, first_query, step_end)
        give = self._passed_pages(request, first_query)
        return all(pool.num_free + g >= n for pool, n, g in zip(self.pools, need, give))

    def can_reserve_all(self, wanted: Sequence[Tuple[Hashable, int, Optional[int]]]) -> bool:
        """Whether reserve() would succeed for every (request, new_len, first_query) of `wanted`,
        one after the other in the order given: all of them, or none, is what a caller needs who
        must not keep pages for some requests when others find none.  The free pages are counted
        along as the calls would leave them: a request is credited the pages its own window has
        passed (reserve gives them back before it takes), never those of a request after it."""
        free = [pool.num_free for pool in self.pools]
        for request, new_len, first_query in wanted:
            need = self.pages_needed(request, new_len, first_query)
            give = self._passed_pages(request, first_query)
            for g in range(len(free)):
                free[g] += give[g]
                if free[g] < need[g]:
                    return False
                free[g] -= need[g]
        return True

    def _passed_pages(self, request, first_query) -> List[int]:
        rc = self.requests[request]
        first_query = rc.num_tokens if first_query is None else first_query
        out = []
        for g, table in enumerate(rc.tables):
            upto = min(self._first_needed_page(g, first_query), len(table))
            out.append(sum(1 for p in table[:upto] if p >= 0 and self.pools[g].ref_count[p] == 1))
        return out

    def reserve(self, request: Hashable, new_len: int, first_query: Optional[int] = None,
                step_end: Optional[int] = None) -> None:
        """Makes the block tables cover positions < new_len (a window group: < step_end, if
        given).  Pages that the window has passed (every position before first_query - window
        + 1) are given back first.  Raises OutOfPages, leaving the request as it was, if a
        pool cannot give enough."""
        rc = self.requests[request]
        first_query = rc.num_tokens if first_query is None else first_query
        if not self.can_reserve(request, new_len, first_query, step_end):
            raise OutOfPages(f"request {request!r}: not enough free pages for {new_len} tokens")
        for g, (pool, table) in enumerate(zip(self.pools, rc.tables)):
            want = self._wanted_pages(g, new_len, step_end)
            first_page = self._first_needed_page(g, first_query)
            for i in range(min(first_page, len(table))):
                if table[i] >= 0:
                    pool.give_back(table[i])
                    table[i] = -1
            while len(table) < want:
                table.append(pool.take() if len(table) >= first_page else -1)
        if step_end is not None and any(group.window is not None for group in self.groups):
            new_len = min(new_len, step_end)                    # positions that every group covers
        rc.num_tokens = max(rc.num_tokens, new_len)

    # ------------------------------------------------------------------ prefix reuse
    def match_prefix(self, tokens: Sequence[int]) -> Tuple[int, List[List[int]]]:
        """How many leading full pages of `tokens` need not be computed, and per group which
        pages stand for them (-1 where a window group needs none).  The chain of hashes is followed
        through every group's pool: n leading pages can be left out if every group that keeps all
        keys still holds all n, and every window group those that the first computed token,
        position n * page_size, still looks at; the largest such n is taken.  The last page of a
        request is never taken from the cache, so that at least one token is computed
        (block_manager.py:62-68)."""
        if not self.prefix_caching:
            return 0, [[] for _ in self.groups]
        ps = self.page_size
        num_pages = (len(tokens) + ps - 1) // ps
        found: List[List[int]] = [[] for _ in self.groups]
        h = -1
        for i in range(num_pages - 1):
            block = tokens[i * ps:(i + 1) * ps]
            h = chain_hash(block, h)
            pages = [pool.lookup(h, block) for pool in self.pools]
            if any(p == -1 and group.window is None for p, group in zip(pages, self.groups)):
                break                       # nothing beyond a page that an all-keys group has lost
            if all(p == -1 for p in pages):
                break
            for g, p in enumerate(pages):
                found[g].append(p)
        hits = 0
        for n in range(len(found[0]), 0, -1):
            if all(-1 not in found[g][self._first_needed_page(g, n * ps):n] for g in range(len(self.groups))):
                hits = n
                break
        return hits, [[p if i >= self._first_needed_page(g, hits * ps) else -1 for i, p in enumerate(found[g][:hits])]
                      for g in range(len(self.groups))]

    def can_admit(self, tokens: Sequence[int], first_step: Optional[int] = None) -> int:
        """-1 if the pages for all of `tokens` are not free, else the number of leading pages
        found in the cache (block_manager.py:58-73): a hit on a page in use costs no free
        page, a hit on a free page still takes it off the free list.  A window group needs the
        pages of the first step's tokens only (first_step of them, default all)."""
        hits, pages = self.match_prefix(tokens)
        step_end = None if first_step is None else hits * self.page_size + first_step
        for g, pool in enumerate(self.pools):
            need = self._wanted_pages(g, len(tokens), step_end) - hits
            need += sum(1 for p in pages[g] if p >= 0 and pool.is_free(p))
            if pool.num_free < need:
                return -1
        if self.slots.num_slots and not self.slots.num_free:
            return -1
        return hits

    def admit_with_prefix(self, request: Hashable, tokens: Sequence[int], first_step: Optional[int] = None) -> int:
        """Admits a request, shares the cached leading pages of `tokens` and reserves the
        rest (block_manager.py:75-92); a window group reserves the first step's tokens only
        (first_step of them, default all).  Returns the number of tokens already in the cache."""
        hits, pages = self.match_prefix(tokens)
        rc = self.admit(request)
        try:
            for pool, table, shared in zip(self.pools, rc.tables, pages):
                for page in shared:
                    if page >= 0:
                        pool.share(page)
                    table.append(page)
            h = -1
            for i in range(hits):
                h = chain_hash(tokens[i * self.page_size:(i + 1) * self.page_size], h)
                rc.hashes.append(h)
            cached = hits * self.page_size
            rc.num_tokens = cached
            self.reserve(request, len(tokens), first_query=cached,
                         step_end=None if first_step is None else cached + first_step)
        except Exception:
            self.release(request)
            raise
        return cached

    def register_full_pages(self, request: Hashable, tokens: Sequence[int], computed: int) -> None:
        """After a step: pages of the request that are now wholly computed get their chained
        hash in every group that still holds them, so that later requests find them
        (block_manager.py:110-120).  `computed` is the number of the request's leading tokens
        whose keys are in the cache."""
        if not self.prefix_caching:
            return
        rc = self.requests[request]
        ps = self.page_size
        for i in range(len(rc.hashes), computed // ps):
            block = tokens[i * ps:(i + 1) * ps]
            h = chain_hash(block, rc.hashes[-1] if rc.hashes else -1)
            rc.hashes.append(h)
            for pool, table in zip(self.pools, rc.tables):
                if i < len(table) and table[i] >= 0:
                    pool.register(table[i], h, block)

    # ------------------------------------------------------------------ checks
    def check(self) -> None:
        """Raises PageError unless every page is either free or held by exactly as many
        block tables as its reference count says, and every slot likewise."""
        for g, pool in enumerate(self.pools):
            holders: Dict[int, int] = {}
            for rc in self.requests.values():
                seen = set()
                for page in rc.tables[g]:
                    if page >= 0:
                        if page in seen:
                            raise PageError(f"page {page} appears twice in one block table")
                        seen.add(page)
                        holders[page] = holders.get(page, 0) + 1
            pool.check(holders)
        held = sorted(rc.state_slot for rc in self.requests.values() if rc.state_slot >= 0)
        if len(held) != len(set(held)):
            raise PageError("a state slot is held by two requests")
        if self.slots.num_slots and len(held) + self.slots.num_free != self.slots.num_slots:
            raise PageError("state slots were lost")
