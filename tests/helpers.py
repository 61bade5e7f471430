"""Shared by the tests: tiny configurations, model folders, and the four ways of driving a
request through the step function (whole; most of it then the last tokens one by one; in
portions of changing size; mixed with other requests on few pages)."""
from __future__ import annotations

import os
import random
import tempfile
from typing import Dict, List, Sequence

import torch

from nano_vllm_amd.config import Qwen3Config
from nano_vllm_amd.engine.batch import StepEntry
from nano_vllm_amd.engine.runner import ModelRunner
from nano_vllm_amd.weights import write_random_model

import plain_qwen3 as plain

# Five tiny configurations; together they differ in every size and option:
# layers, width, heads and groups, head size, inner size, vocabulary, theta, eps, tying,
# norm weights, page size, and (e) a bias on q/k/v, which takes the per-head q/k norm away
# (nanovllm/models/qwen3.py:40-48,68-70).
CONFIGS: Dict[str, dict] = {
    "a": dict(cfg=Qwen3Config(vocab_size=256, hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
                              num_key_value_heads=2, head_dim=16, intermediate_size=128, rms_norm_eps=1e-6,
                              rope_theta=10000.0, max_position_embeddings=128, tie_word_embeddings=True),
              norm_std=0.0, page=4, seed=11),
    "b": dict(cfg=Qwen3Config(vocab_size=384, hidden_size=96, num_hidden_layers=3, num_attention_heads=8,
                              num_key_value_heads=2, head_dim=32, intermediate_size=160, rms_norm_eps=1e-5,
                              rope_theta=1000000.0, max_position_embeddings=256, tie_word_embeddings=False),
              norm_std=0.1, page=8, seed=12),
    "c": dict(cfg=Qwen3Config(vocab_size=1000, hidden_size=120, num_hidden_layers=2, num_attention_heads=6,
                              num_key_value_heads=3, head_dim=64, intermediate_size=200, rms_norm_eps=1e-6,
                              rope_theta=500000.0, max_position_embeddings=1024, tie_word_embeddings=False),
              norm_std=0.1, page=16, seed=13),
    "d": dict(cfg=Qwen3Config(vocab_size=777, hidden_size=256, num_hidden_layers=2, num_attention_heads=8,
                              num_key_value_heads=2, head_dim=128, intermediate_size=384, rms_norm_eps=1e-6,
                              rope_theta=1000000.0, max_position_embeddings=2048, tie_word_embeddings=True),
              norm_std=0.05, page=64, seed=14),
    # the biases are made ten times larger than N(0, 0.02) draws them, as large as the products
    # they are added to, so that a bias left out or added twice moves every logit
    "e": dict(cfg=Qwen3Config(vocab_size=300, hidden_size=80, num_hidden_layers=2, num_attention_heads=4,
                              num_key_value_heads=1, head_dim=32, intermediate_size=144, rms_norm_eps=1e-5,
                              rope_theta=50000.0, max_position_embeddings=512, tie_word_embeddings=False,
                              attention_bias=True),
              norm_std=0.1, page=16, seed=15, bias_scale=10.0),
}

_folders: Dict[str, str] = {}
_tmp = None


def model_folder(name: str, dtype: str = "float32") -> str:
    """A folder with config.json and model.safetensors of the named tiny configuration,
    written once per test session into a temporary folder."""
    global _tmp
    key = f"{name}-{dtype}"
    if key not in _folders:
        if _tmp is None:
            _tmp = tempfile.TemporaryDirectory(prefix="nva-models-")
        c = CONFIGS[name]
        path = os.path.join(_tmp.name, key)
        write_random_model(path, c["cfg"], seed=c["seed"], norm_std=c["norm_std"], dtype=dtype)
        if c.get("bias_scale"):
            from safetensors.torch import load_file, save_file
            file = os.path.join(path, "model.safetensors")
            tensors = load_file(file)
            assert any(k.endswith(".bias") for k in tensors)
            tensors = {k: (t.float() * c["bias_scale"]).to(t.dtype) if k.endswith(".bias") else t
                       for k, t in tensors.items()}
            save_file(tensors, file, metadata={"format": "pt"})
        _folders[key] = path
    return _folders[key]


def random_tokens(vocab: int, n: int, seed: int) -> List[int]:
    rng = random.Random(seed)
    return [rng.randrange(vocab) for _ in range(n)]


def make_runner(folder: str, dtype: str, page: int, num_pages: int, device="cuda:0", kernels=None,
                max_requests: int = 8, prefix_caching: bool = False) -> ModelRunner:
    return ModelRunner.from_folder(folder, dtype=dtype, device=device, page_size=page, num_pages=num_pages,
                                   max_requests=max_requests, kernels=kernels, quiet=True,
                                   enable_prefix_caching=prefix_caching)


# ------------------------------------------------------------------------------ drivings
def run_portions(runner: ModelRunner, rid, tokens: Sequence[int], portions: Sequence[int]) -> torch.Tensor:
    """One request alone, cut into the given portions; logits of every position."""
    assert sum(portions) == len(tokens)
    runner.cache.admit(rid)
    out, pos = [], 0
    for n in portions:
        runner.cache.reserve(rid, pos + n)
        out.append(runner.step([StepEntry(rid, tokens[pos:pos + n], pos, list(range(n)))]).float().cpu())
        pos += n
    runner.cache.release(rid)
    runner.cache.check()
    return torch.cat(out)


def whole(n: int) -> List[int]:
    return [n]


def last_one_by_one(n: int, last: int = 32) -> List[int]:
    last = min(last, n - 1)
    return [n - last] + [1] * last


def changing_portions(n: int, seed: int) -> List[int]:
    """Portions of changing size, down to two tokens (and ones at the end)."""
    rng = random.Random(seed)
    sizes, left = [], n
    menu = [7, 2, 16, 3, 2, 33, 5, 2, 64, 9]
    i = rng.randrange(len(menu))
    while left > 0:
        s = min(menu[i % len(menu)], left)
        sizes.append(s)
        left -= s
        i += 1
    return sizes


def run_mixed(runner: ModelRunner, requests: Dict[str, List[int]], seed: int, max_live: int = 4):
    """Up to max_live requests at a time: portions of some beside single decoded tokens of
    others; a request that ends gives its pages back and a waiting one takes them.  Returns
    {request: logits of every position}."""
    rng = random.Random(seed)
    waiting = list(requests)
    live: Dict[str, int] = {}
    got: Dict[str, List[torch.Tensor]] = {r: [] for r in requests}
    decoding = set()
    while waiting or live:
        while waiting and len(live) < max_live:
            rid = waiting[0]
            need = len(requests[rid])
            pages_needed = (need + runner.page_size - 1) // runner.page_size
            if runner.cache.pools[0].num_free - _reserved_pages(runner, live, requests) < pages_needed:
                break
            waiting.pop(0)
            runner.cache.admit(rid)
            live[rid] = 0
        assert live, "the pool is too small for any request"
        entries = []
        for rid, pos in live.items():
            left = len(requests[rid]) - pos
            if rid in decoding or left <= 32:
                decoding.add(rid)
                n = 1
            else:
                n = min(left - 32, rng.choice([2, 3, 5, 8, 13, 21, 40]))
            runner.cache.reserve(rid, pos + n)
            entries.append(StepEntry(rid, requests[rid][pos:pos + n], pos, list(range(n))))
        rng.shuffle(entries)
        logits = runner.step(entries).float().cpu()
        row = 0
        for e in entries:
            n = len(e.tokens)
            got[e.request].append(logits[row:row + n])
            row += n
            live[e.request] += n
            if live[e.request] == len(requests[e.request]):
                runner.cache.release(e.request)
                del live[e.request]
                decoding.discard(e.request)
        runner.cache.check()
    return {r: torch.cat(v) for r, v in got.items()}


def run_mixed_with_prefix_reuse(runner: ModelRunner, requests: Dict[str, List[int]], seed: int, max_live: int = 3):
    """As run_mixed, with the cache manager's prefix reuse on, driven as the scheduler drives
    it: a request is admitted when all its pages are free, takes the leading pages that
    earlier requests left under their hashes (in use or already given back) and runs only
    the tokens after them; after every step its full pages are registered.  Returns
    ({request: (first computed position, logits from there on)}, counts of the hits)."""
    rng = random.Random(seed)
    cache = runner.cache
    assert cache.prefix_caching
    waiting = list(requests)
    live: Dict[str, int] = {}
    first: Dict[str, int] = {}
    got: Dict[str, List[torch.Tensor]] = {r: [] for r in requests}
    stats = {"hit_in_use": 0, "hit_given_back": 0, "pages_taken": 0, "admitted_without_hit": 0, "finished": []}
    while waiting or live:
        while waiting and len(live) < max_live:
            rid = waiting[0]
            toks = requests[rid]
            if cache.can_admit(toks) == -1:
                break
            pages = cache.match_prefix(toks)[1][0]
            for p in pages:
                stats["hit_given_back" if cache.pools[0].is_free(p) else "hit_in_use"] += 1
            if not pages:
                stats["admitted_without_hit"] += 1
            waiting.pop(0)
            cached = cache.admit_with_prefix(rid, toks)
            assert cached == len(pages) * runner.page_size and cached < len(toks)
            stats["pages_taken"] += len(cache.table(rid, 0)) - len(pages)
            live[rid] = first[rid] = cached
        assert live, "the pool is too small for any request"
        entries = []
        for rid, pos in live.items():
            left = len(requests[rid]) - pos
            n = 1 if left <= 12 else min(left - 12, rng.choice([2, 3, 5, 8, 13, 21, 40]))
            entries.append(StepEntry(rid, requests[rid][pos:pos + n], pos, list(range(n))))
        rng.shuffle(entries)
        logits = runner.step(entries).float().cpu()
        row = 0
        for e in entries:
            n = len(e.tokens)
            got[e.request].append(logits[row:row + n])
            row += n
            live[e.request] += n
            cache.register_full_pages(e.request, requests[e.request], live[e.request])
            if live[e.request] == len(requests[e.request]):
                cache.release(e.request)
                del live[e.request]
                stats["finished"].append(e.request)
        cache.check()
    return {r: (first[r], torch.cat(v)) for r, v in got.items()}, stats


def prefix_requests(name: str, top: int) -> Dict[str, Dict[str, List[int]]]:
    """Requests for the drive with prefix reuse, in three phases that run one after the other on
    the same pool.  share: three requests with a common prefix of five pages and a token (and
    tails of their own) among others that share nothing.  churn: requests that together take
    more pages than the pool has, so that every hashed page is taken again.  again: the common
    prefix once more (it is gone and is computed again), then that whole request with eleven
    tokens added (all its full pages are found)."""
    c = CONFIGS[name]
    V, page = c["cfg"].vocab_size, c["page"]
    shared = random_tokens(V, 5 * page + 1, 90)
    fill = lambda n, s: random_tokens(V, n, s)
    share = {"s0": shared + fill(top // 4, 91), "f1": fill(top // 2, 92), "f2": fill(top // 3 + 5, 93),
             "s3": shared + fill(top // 3, 94), "s4": shared + fill(9, 95)}
    churn = {f"f{i}": fill(top - 10 * i, 90 + i) for i in range(5, 9)}
    s9 = shared + fill(top // 5, 99)
    return {"share": share, "churn": churn, "again": {"s9": s9}, "again2": {"s10": s9 + fill(11, 100)}}


def prefix_pool_pages(name: str, top: int) -> int:
    """A pool for about two of the largest requests of prefix_requests."""
    page = CONFIGS[name]["page"]
    need = sorted(((len(t) + page - 1) // page for phase in prefix_requests(name, top).values()
                   for t in phase.values()), reverse=True)
    return need[0] + need[1]


def check_prefix_reuse(runner: ModelRunner, name: str, top: int, plain_of, tol: float, seed: int = 6):
    """The drive with prefix reuse and its checks, for the GPU and for the host-only test:
    plain_of(tokens) gives the plain logits of a whole request."""
    page = CONFIGS[name]["page"]
    phases = prefix_requests(name, top)
    pool = runner.cache.pools[0]

    def drive(reqs):
        got, stats = run_mixed_with_prefix_reuse(runner, reqs, seed=seed)
        for rid, toks in reqs.items():
            first, logits = got[rid]
            want = plain_of(toks)[first:]
            assert logits.shape == want.shape
            assert rel_err(logits, want) < tol, (rid, first)
        assert pool.num_free == pool.num_pages
        return {r: got[r][0] for r in reqs}, stats

    firsts, stats = drive(phases["share"])
    # s3 and s4 come when s0 has registered the prefix: its pages are found in use or given back
    assert firsts["s0"] == 0 and firsts["s3"] == firsts["s4"] == 5 * page, firsts
    assert stats["hit_in_use"] > 0 and stats["hit_given_back"] > 0, stats
    churn_pages = sum((len(t) + page - 1) // page for t in phases["churn"].values())
    assert churn_pages >= pool.num_pages
    firsts, stats = drive(phases["churn"])
    assert stats["pages_taken"] >= pool.num_pages, stats       # from the head of the free list: every page once at least
    firsts, stats = drive(phases["again"])
    assert firsts["s9"] == 0 and stats["admitted_without_hit"] == 1      # every hashed page was taken again
    firsts, stats = drive(phases["again2"])
    full = len(phases["again"]["s9"]) // page
    assert firsts["s10"] == full * page and stats["hit_given_back"] == full, (firsts, stats)


def _reserved_pages(runner, live, requests) -> int:
    """Pages that live requests will still take before they end."""
    total = 0
    for rid, pos in live.items():
        full = (len(requests[rid]) + runner.page_size - 1) // runner.page_size
        total += full - len(runner.cache.table(rid, 0))
    return total


def plain_logits(folder: str, tokens: Sequence[int], rounding=None) -> torch.Tensor:
    cfg, w = plain.read_folder(folder)
    return plain.logits(w, cfg, list(tokens), rounding)


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    return float((got.double() - want.double()).abs().max() / want.double().abs().max())


def run_mixed_groups(runner: ModelRunner, requests: Dict[str, List[int]], seed: int, max_live: int = 4):
    """As run_mixed for models with several cache groups: a request is admitted when every
    group can take its first portion, and a portion that finds no pages waits for a step."""
    rng = random.Random(seed)
    waiting = list(requests)
    live: Dict[str, int] = {}
    got: Dict[str, List[torch.Tensor]] = {r: [] for r in requests}
    for _ in range(100000):
        if not waiting and not live:
            break
        while waiting and len(live) < max_live:
            rid = waiting.pop(0)
            runner.cache.admit(rid)
            live[rid] = 0
        entries = []
        for rid, pos in live.items():
            left = len(requests[rid]) - pos
            n = 1 if left <= 20 else min(left - 20, rng.choice([2, 3, 5, 8, 13, 21]))
            if not runner.cache.can_reserve(rid, pos + n, first_query=pos):
                n = 1
                if not runner.cache.can_reserve(rid, pos + 1, first_query=pos):
                    continue
            runner.cache.reserve(rid, pos + n, first_query=pos)
            entries.append(StepEntry(rid, requests[rid][pos:pos + n], pos, list(range(n))))
        assert entries, "no request can go on: the pools are too small"
        rng.shuffle(entries)
        logits = runner.step(entries).float().cpu()
        row = 0
        for e in entries:
            n = len(e.tokens)
            got[e.request].append(logits[row:row + n])
            row += n
            live[e.request] += n
            if live[e.request] == len(requests[e.request]):
                runner.cache.release(e.request)
                del live[e.request]
        runner.cache.check()
    return {r: torch.cat(v) for r, v in got.items()}
