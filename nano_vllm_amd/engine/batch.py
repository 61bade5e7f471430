"""A step's batch: requests with their next tokens, flattened for the kernels.

Reference: prepare_prefill / prepare_decode of nanovllm/engine/model_runner.py:129-188 and the
Context of nanovllm/utils/context.py:5-27.  Here one description covers every mixture:
entries with one token (decoding) come first, portions of prompts after them; each token
carries its request's index and its absolute position, each request the number of keys it
sees (tokens in the cache after this step) and its block table per cache group.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch


@dataclass
class StepEntry:
    request: Hashable
    tokens: Sequence[int]            # the tokens this step runs for the request
    start: int                       # absolute position of tokens[0] = tokens already in the cache
    want: Sequence[int] = ()         # places among `tokens` whose logits are wanted


@dataclass
class GroupBatch:
    block_tables: torch.Tensor       # int32 [S, pages]; -1: no page
    slot_mapping: torch.Tensor       # int32 [T]: page * page_size + offset of each token's key


@dataclass
class StepBatch:
    num_tokens: int
    num_seqs: int
    num_decode: int                  # leading requests that bring exactly one token
    input_ids: torch.Tensor          # int32 [T]
    positions: torch.Tensor          # int32 [T] absolute positions
    token_seq: torch.Tensor          # int32 [T] index of the token's request in this batch
    cu_seqlens_q: torch.Tensor       # int32 [S+1]
    kv_lens: torch.Tensor            # int32 [S] keys each request sees = start + its tokens
    seq_starts: torch.Tensor         # int32 [S] tokens each request had in the cache before
    state_slots: torch.Tensor        # int32 [S]
    logits_rows: Optional[torch.Tensor]   # int32 [R] flat token indices, in the caller's order
    groups: List[GroupBatch]
    max_q_len: int
    max_kv_len: int
    # host copies
    q_lens: List[int] = field(default_factory=list)
    starts: List[int] = field(default_factory=list)
    requests: List[Hashable] = field(default_factory=list)
    step_cache: dict = field(default_factory=dict)   # emptied by the model at the start of every pass
    # int32 lists that the kernels asked to have uploaded with the batch (name -> device tensor);
    # the batch builder does not know what they mean
    extras: Dict[str, torch.Tensor] = field(default_factory=dict)


def build_batch(entries: Sequence[StepEntry], cache, page_size: int, vocab_size: int, device,
                table_width: Optional[int] = None, static: Optional[torch.Tensor] = None,
                pad_to: Optional[int] = None, max_position: Optional[int] = None,
                extras: Optional[Callable[[List[int], List[int], int], Dict[str, List[int]]]] = None) -> StepBatch:
    """Orders the entries (single tokens first), checks them against the cache manager's
    block tables and uploads everything in one copy.

    table_width fixes the width of the block tables (else: the widest table of the batch).
    static, an int32 device tensor of the batch's flat size, receives the copy instead of a
    new tensor: with equal counts of tokens, requests and wanted places and a fixed table
    width the layout is the same for every step, which is what a captured graph replays on.
    pad_to (decoded tokens only) fills the batch up to that many requests with copies of the
    first entry that write nothing into the cache (slot -1): they read what the first request
    reads, and their logits, which follow the real ones, are dropped by the caller; where requests
    hold state slots, theirs is the spare slot after the requests' own.
    max_position: the positions the model knows (rows of its position tables); an entry that
    reaches beyond is refused here, since the kernels read those tables unchecked.
    extras(q_lens, starts, num_decode) -> {name: [int, ...]}: lists that depend on the step's
    shape only and that the kernels want on the device; they travel in the same copy and come
    back as StepBatch.extras[name] (flat int32)."""
    if not entries:
        raise ValueError("a step needs at least one entry")
    order = sorted(range(len(entries)), key=lambda i: (len(entries[i].tokens) != 1, i))
    offsets = {}
    t = 0
    for i in order:
        offsets[i] = t
        t += len(entries[i].tokens)
    T, S = t, len(entries)
    num_groups = len(cache.groups)

    # per request a few arrays (a portion of a prompt has thousands of tokens: no Python per token)
    input_ids, positions, token_seq = [], [], []
    cu, kv_lens, starts, state_slots, q_lens = [0], [], [], [], []
    slot_maps = [[] for _ in range(num_groups)]
    tables = [[] for _ in range(num_groups)]
    one_ids, one_pos, one_slots = [], [], [[] for _ in range(num_groups)]
    seen = set()
    for s, i in enumerate(order):
        e = entries[i]
        n = len(e.tokens)
        if n == 0:
            raise ValueError(f"request {e.request!r} brings no token")
        if e.request in seen:
            raise ValueError(f"request {e.request!r} appears twice in one step")
        seen.add(e.request)
        rc = cache.requests[e.request]
        if e.start < 0 or e.start + n > rc.num_tokens:
            raise ValueError(f"request {e.request!r}: positions {e.start}..{e.start + n - 1} are not reserved "
                             f"in the cache ({rc.num_tokens} are)")
        if max_position is not None and e.start + n > max_position:
            raise ValueError(f"request {e.request!r}: position {e.start + n - 1} is beyond the model's "
                             f"{max_position} positions (max_position_embeddings)")
        cu.append(cu[-1] + n)
        kv_lens.append(e.start + n)
        starts.append(e.start)
        q_lens.append(n)
        state_slots.append(rc.state_slot)
        if n == 1:                                   # a decoded token (these come first): plain integers
            tok = e.tokens[0]
            if not 0 <= tok < vocab_size:
                raise ValueError(f"request {e.request!r}: token id {tok} is outside the vocabulary of {vocab_size}")
            one_ids.append(tok)
            one_pos.append(e.start)
            for g in range(num_groups):
                table = rc.tables[g]
                tables[g].append(table)
                page = table[e.start // page_size]
                if page < 0:
                    raise ValueError(f"request {e.request!r}: position {e.start} has no page in group {g}")
                one_slots[g].append(page * page_size + e.start % page_size)
            continue
        toks = np.asarray(e.tokens, dtype=np.int64)
        if toks.ndim != 1 or int(toks.min()) < 0 or int(toks.max()) >= vocab_size:
            bad = next(int(tok) for tok in e.tokens if not 0 <= tok < vocab_size)
            raise ValueError(f"request {e.request!r}: token id {bad} is outside the vocabulary of {vocab_size}")
        pos = np.arange(e.start, e.start + n, dtype=np.int64)
        input_ids.append(toks)
        positions.append(pos)
        token_seq.append(np.full(n, s, dtype=np.int64))
        for g in range(num_groups):
            table = rc.tables[g]
            tables[g].append(table)
            pages = np.asarray(table, dtype=np.int64)[pos // page_size]
            if int(pages.min()) < 0:
                where = int(pos[int(np.argmax(pages < 0))])
                raise ValueError(f"request {e.request!r}: position {where} has no page in group {g}")
            slot_maps[g].append(pages * page_size + pos % page_size)
    num_decode = len(one_ids)
    pad = 0
    if pad_to is not None and pad_to > S:
        if num_decode != S:
            raise ValueError("only a batch of decoded tokens can be padded")
        pad = pad_to - S
        one_ids += [one_ids[0]] * pad
        one_pos += [one_pos[0]] * pad
        for values in (kv_lens, starts, q_lens):
            values += [values[0]] * pad
        # state: the spare slot that no request holds (the state tensors' last row), so that a mixer
        # may read and write the padding rows' state like any other
        state_slots += [cache.slots.num_slots if cache.slots.num_slots else state_slots[0]] * pad
        cu += list(range(S + 1, S + pad + 1))
        for g in range(num_groups):
            one_slots[g] += [-1] * pad
            tables[g] += [tables[g][0]] * pad
        T, S, num_decode = T + pad, S + pad, num_decode + pad
    rows = []
    for i, e in enumerate(entries):
        for w in e.want:
            if not 0 <= w < len(e.tokens):
                raise ValueError(f"request {e.request!r}: wanted place {w} is outside its {len(e.tokens)} tokens")
            rows.append(offsets[i] + w)
    rows += list(range(T - pad, T))

    widths = [max(1, max(len(tb) for tb in tables[g])) for g in range(num_groups)]
    if table_width is not None:
        if max(widths, default=1) > table_width:
            raise ValueError(f"a block table of {max(widths)} pages exceeds the fixed width {table_width}")
        widths = [table_width] * num_groups
    extra_lists = dict(extras(q_lens, starts, num_decode)) if extras is not None else {}
    scalars = cu + kv_lens + starts + state_slots + rows
    for values in extra_lists.values():
        scalars = scalars + list(values)
    if num_decode == S:                              # decoded tokens only: one list, one conversion
        flat: List[int] = one_ids + one_pos + list(range(S)) + scalars
        for g in range(num_groups):
            flat += one_slots[g]
            for tb in tables[g]:
                flat += tb
                flat += [-1] * (widths[g] - len(tb))
        host = torch.tensor(flat, dtype=torch.int32)
    else:
        as_array = lambda values: np.asarray(values, dtype=np.int64)
        pieces = [as_array(one_ids)] + input_ids + [as_array(one_pos)] + positions
        pieces += [np.arange(num_decode, dtype=np.int64)] + token_seq + [as_array(scalars)]
        for g in range(num_groups):
            pieces += [as_array(one_slots[g])] + slot_maps[g]
            padded: List[int] = []
            for tb in tables[g]:
                padded += tb
                padded += [-1] * (widths[g] - len(tb))
            pieces.append(as_array(padded))
        host = torch.from_numpy(np.concatenate(pieces).astype(np.int32))
    if static is not None:
        if static.numel() != host.numel():
            raise ValueError("the static batch buffer does not fit this batch's layout")
        static.copy_(host)
        dev = static
    else:
        dev = host.to(device)

    pos = 0

    def take(n):
        nonlocal pos
        out = dev[pos:pos + n]
        pos += n
        return out

    b_ids, b_pos, b_seq = take(T), take(T), take(T)
    b_cu, b_kv, b_starts, b_slots = take(S + 1), take(S), take(S), take(S)
    b_rows = take(len(rows)) if rows else None
    b_extras = {name: take(len(values)) for name, values in extra_lists.items()}
    groups = []
    for g in range(num_groups):
        sm = take(T)
        bt = take(S * widths[g]).view(S, widths[g])
        groups.append(GroupBatch(bt, sm))
    return StepBatch(
        num_tokens=T, num_seqs=S, num_decode=num_decode, extras=b_extras,
        input_ids=b_ids, positions=b_pos, token_seq=b_seq, cu_seqlens_q=b_cu, kv_lens=b_kv,
        seq_starts=b_starts, state_slots=b_slots, logits_rows=b_rows, groups=groups,
        max_q_len=max(q_lens), max_kv_len=max(kv_lens), q_lens=q_lens, starts=starts,
        requests=[entries[i].request for i in order])
