"""The engine loop and the Python entry point's methods.

Reference: nanovllm/engine/llm_engine.py:15-90 - LLMEngine(model, **config), add_request,
step, is_finished, generate - with the same names and meanings.  Differences: unknown
keyword arguments are an error instead of being dropped; prompts of token ids need no
tokenizer, and "text" is None where none is available; temperature 0 is greedy.
"""
from __future__ import annotations

import os
import sys
from time import perf_counter
from typing import Dict, List, Optional, Sequence as Seq, Tuple, Union

import torch

from ..config.engine_config import EngineConfig
from ..sampling.params import SamplingParams
from ..sampling.sampler import Sampler
from .batch import StepEntry
from .runner import ModelRunner, load_model
from .scheduler import Scheduler
from .sequence import Sequence


class LLMEngine:
    def __init__(self, model: str, kernels=None, **kwargs):
        """kernels: None for the HIP kernels (the only implementation in the package), or an
        object with the same operations, which tests use to run the host logic elsewhere."""
        unknown = set(kwargs) - EngineConfig.field_names()
        if unknown:
            raise TypeError(f"unknown engine options {sorted(unknown)}; known: {sorted(EngineConfig.field_names())}")
        self.config = cfg = EngineConfig(model, **kwargs)
        self.model = load_model(cfg.model, cfg.dtype, cfg.device, kernels, random_weights=cfg.random_weights)
        spec = self.model.spec
        cfg.max_model_len = min(cfg.max_model_len, spec.max_position)           # config.py:25
        num_pages = cfg.num_kvcache_blocks          # one count for every cache group, or a list with one per group
        if num_pages is None or (not isinstance(num_pages, (list, tuple)) and num_pages <= 0):
            num_pages = self._pages_from_free_memory()
            cfg.num_kvcache_blocks = num_pages
        self.runner = ModelRunner(self.model, cfg.kvcache_block_size, num_pages, cfg.max_num_seqs,
                                  enable_prefix_caching=cfg.enable_prefix_caching)
        if not cfg.enforce_eager and self.model.device.type == "cuda":
            self.runner.enable_decode_graphs(min(cfg.max_num_seqs, 512), cfg.max_model_len,
                                             measure_products=cfg.measure_products)
            self.runner.capture_decode_graphs()          # at start-up, as the reference does (model_runner.py:222)
        eos = [cfg.eos] if cfg.eos >= 0 else list(spec.eos_token_ids) or self._eos_from_generation_config()
        self.tokenizer = None
        self.scheduler = Scheduler(self.runner.cache, cfg.max_num_seqs, cfg.max_num_batched_tokens,
                                   cfg.max_model_len, eos, cfg.schedule)
        self.sampler = Sampler(self.model.kernels, self.model.device)
        self.stats = {"prefill_tokens": 0, "prefill_time": 0.0, "decode_tokens": 0, "decode_time": 0.0, "steps": 0}
        self._by_id: Dict[int, Sequence] = {}
        self._next_id = 0

    # ------------------------------------------------------------------ set-up helpers
    def _pages_from_free_memory(self) -> int:
        """As nanovllm/engine/model_runner.py:91-114: the largest step the options allow is run
        once (max_num_batched_tokens prompt tokens in requests of up to max_model_len), on a
        cache just large enough for it, and the most device memory it held beside weights and
        cache is measured; the pages are what gpu_memory_utilization of the device leaves after
        everything in use now, that peak, and what the captured decode steps keep."""
        from ..cache import storage
        from ..cache.manager import plan_groups
        cfg, model = self.config, self.model
        if model.device.type != "cuda":
            raise RuntimeError("num_kvcache_blocks must be given when the model is not on a GPU")
        needs = model.cache_needs()
        groups, state_runs = plan_groups(needs)
        itemsize = torch.empty((), dtype=model.dtype).element_size()
        per_page = sum(storage.bytes_per_page(needs, groups, cfg.kvcache_block_size, itemsize))
        step_peak = self._largest_step_peak()
        torch.cuda.empty_cache()
        free, total = torch.cuda.mem_get_info(model.device)
        used = total - free
        kept = 0
        if not cfg.enforce_eager:
            # every captured decode step keeps its own logits: one row per request of its batch size
            top = min(cfg.max_num_seqs, 512)
            rows = sum({ModelRunner.graph_batch_size(n) for n in range(1, top + 1)})
            kept = rows * model.spec.vocab_size * 4
        kept += cfg.max_num_seqs * storage.state_bytes_per_slot(needs, state_runs)
        budget = int(total * cfg.gpu_memory_utilization) - used - step_peak - kept
        pages = budget // max(per_page, 1)
        if pages <= 0:
            raise RuntimeError("no device memory is left for the cache (model_runner.py:114)")
        self.warmup_peak_bytes = step_peak
        return int(pages)

    def _largest_step_peak(self) -> int:
        """Bytes the largest step holds at its peak beyond what was allocated before it (weights and
        cache): the step is run on a runner of its own whose cache holds just its tokens
        (model_runner.py:91-101 runs it before the cache exists)."""
        cfg, model = self.config, self.model
        per_request = max(1, min(cfg.max_model_len - 1, cfg.max_num_batched_tokens))
        lengths = []
        left = cfg.max_num_batched_tokens
        while left > 0 and len(lengths) < cfg.max_num_seqs:
            lengths.append(min(per_request, left))
            left -= lengths[-1]
        page = cfg.kvcache_block_size
        pages = sum((n + page - 1) // page for n in lengths)
        runner = ModelRunner(model, page, pages, len(lengths), enable_prefix_caching=False)
        try:
            entries = []
            for i, n in enumerate(lengths):
                name = ("warm-up", i)
                runner.cache.admit(name)
                runner.cache.reserve(name, n)
                entries.append(StepEntry(name, [0] * n, 0, [n - 1]))
            torch.cuda.synchronize(model.device)
            torch.cuda.reset_peak_memory_stats(model.device)
            before = torch.cuda.memory_allocated(model.device)
            logits = runner.step(entries)
            Sampler(model.kernels, model.device).sample(logits, [1.0] * len(lengths), [0] * len(lengths), list(range(len(lengths))), lengths)
            torch.cuda.synchronize(model.device)
            peak = torch.cuda.max_memory_allocated(model.device) - before
            del logits
        finally:
            del runner
        return max(int(peak), 0)

    def _eos_from_generation_config(self) -> List[int]:
        path = os.path.join(self.config.model, "generation_config.json")
        if os.path.isfile(path):
            import json
            with open(path) as f:
                eos = json.load(f).get("eos_token_id")
            if isinstance(eos, int):
                return [eos]
            if isinstance(eos, list):
                return [int(e) for e in eos]
        return []

    def _tokenizer(self):
        if self.tokenizer is None:
            try:
                from transformers import AutoTokenizer      # llm_engine.py:32
                self.tokenizer = AutoTokenizer.from_pretrained(self.config.model, use_fast=True)
            except Exception as e:
                raise RuntimeError(f"a text prompt needs a tokenizer in {self.config.model!r}: {e}") from e
        return self.tokenizer

    # ------------------------------------------------------------------ the reference's methods
    def add_request(self, prompt: Union[str, List[int]], sampling_params: Optional[SamplingParams] = None) -> int:
        if isinstance(prompt, str):
            prompt = self._tokenizer().encode(prompt)
        seq = Sequence(list(prompt), sampling_params, seq_id=self._next_id)
        self._next_id += 1
        self.scheduler.add(seq)
        self._by_id[seq.seq_id] = seq
        return seq.seq_id

    def is_finished(self) -> bool:
        return self.scheduler.is_finished()

    def step(self) -> Tuple[List[Tuple[int, List[int]]], int]:
        """One scheduling decision and one model step.  Returns the requests finished in it
        as (id, completion token ids), and the token count of the step: positive for a step
        of prompt tokens, minus the number of decoded tokens for a decode step (llm_engine.py:49-55:
        one per request; here times the steps of a burst)."""
        t0 = perf_counter()
        seqs, is_prefill = self.scheduler.schedule()
        num_tokens = 0
        if seqs:
            entries, sampled, decoding = [], [], []
            for seq in seqs:
                start, n = seq.num_cached_tokens, seq.num_scheduled_tokens
                last = start + n == seq.num_tokens
                decoding.append(n == 1 and last and seq.num_completion_tokens > 0)
                entries.append(StepEntry(seq.seq_id, seq.token_ids[start:start + n], start, [n - 1] if last else []))
                if last:
                    sampled.append(seq)
            burst = self._burst_steps(seqs, entries, is_prefill)
            decoded = len(seqs)                  # tokens a decode step reports: one per request and step of a burst that it is still in
            if burst > 1:
                rows = self.runner.decode_burst(
                    entries, burst, self.sampler, [s.temperature for s in seqs],
                    [self.config.seed if s.seed is None else s.seed for s in seqs], [s.seq_id for s in seqs])
                for row in rows:                 # as after `burst` single steps; what follows a request's end is dropped
                    live = [(s, t) for s, t in zip(seqs, row) if not s.is_finished]
                    for s, _ in live:
                        s.num_scheduled_tokens = 1
                    self.scheduler.postprocess([s for s, _ in live], [t for _, t in live])
                    self.stats["decode_tokens"] += len(live)
                    decoded += len(live)
                decoded -= len(seqs)
                self.stats["decode_tokens"] -= len(seqs)            # the first row is counted below
            else:
                logits = self.runner.step(entries)
                tokens = {}
                if sampled:
                    ids = self.sampler.sample(
                        logits, [s.temperature for s in sampled],
                        [self.config.seed if s.seed is None else s.seed for s in sampled],
                        [s.seq_id for s in sampled], [s.num_tokens for s in sampled])
                    tokens = {s.seq_id: t for s, t in zip(sampled, ids)}
                elif self.model.device.type == "cuda":
                    torch.cuda.synchronize(self.model.device)
                self.scheduler.postprocess(seqs, [tokens.get(s.seq_id, -1) for s in seqs])
            num_tokens = sum(len(e.tokens) for e in entries) if is_prefill else -decoded
            dt = perf_counter() - t0
            # tokens by what they are (a mixed step holds both kinds), time by the kind of the step
            self.stats["prefill_tokens"] += sum(len(e.tokens) for e, d in zip(entries, decoding) if not d)
            self.stats["decode_tokens"] += sum(decoding)
            self.stats["prefill_time" if is_prefill else "decode_time"] += dt
            self.stats["steps"] += 1
        finished = self.scheduler.just_finished
        self.scheduler.just_finished = []
        outputs = [(s.seq_id, s.completion_token_ids) for s in finished]
        return outputs, num_tokens

    def _burst_steps(self, seqs, entries, is_prefill) -> int:
        """How many decode steps to run in a row without the host: more than one only while
        no request waits, every request of the step decodes, the captured steps take the batch,
        and pages for all the steps can be reserved."""
        want = self.config.decode_burst
        if want <= 1 or is_prefill or self.scheduler.waiting or not seqs:
            return 1
        runner = self.runner
        if not (getattr(runner, "_graph_max_batch", 0) and runner._graph_takes(entries)):
            return 1
        if len(runner.groups) > getattr(self.model.kernels, "max_burst_groups", 0):
            return 1            # the kernel that advances a step's metadata on the device takes so many groups
        for s in seqs:
            if s.num_cached_tokens + 1 != s.num_tokens:
                return 1
        left = [s.max_tokens - s.num_completion_tokens for s in seqs]
        room = min(self.config.max_model_len - s.num_tokens for s in seqs)
        # A burst may run past the last token of some of its requests, as it runs past an eos token:
        # their rows are computed and dropped, and the host is asked once per burst and not once per
        # request that ends.  It never runs past the last token of all of them, nor past the longest
        # sequence the model takes; where the pool has no pages for that, it ends with the first
        # request that ends.
        for steps in dict.fromkeys((min(want, max(left), room), min(want, min(left), room))):
            if steps <= 1:
                break
            # all requests or none: a request must not keep pages for steps that will not run
            wanted = [(s.seq_id, s.num_tokens + steps - 1, s.num_tokens - 1) for s in seqs]
            if runner.cache.can_reserve_all(wanted):
                for request, new_len, first_query in wanted:
                    runner.cache.reserve(request, new_len, first_query=first_query)
                return steps
        return 1

    def generate(self, prompts: Seq[Union[str, List[int]]],
                 sampling_params: Union[SamplingParams, Seq[SamplingParams], None] = None,
                 use_tqdm: bool = True) -> List[dict]:
        """llm_engine.py:60-90: returns, in the order of the prompts, {"text", "token_ids"}."""
        if sampling_params is None:
            sampling_params = SamplingParams()
        if not isinstance(sampling_params, (list, tuple)):
            sampling_params = [sampling_params] * len(prompts)
        ids = [self.add_request(p, sp) for p, sp in zip(prompts, sampling_params)]
        done: Dict[int, List[int]] = {}
        prefill_tps = decode_tps = 0.0
        last_print = perf_counter()
        while not self.is_finished():
            t = perf_counter()
            outputs, n = self.step()
            dt = max(perf_counter() - t, 1e-9)
            if n > 0:
                prefill_tps = n / dt
            elif n < 0:
                decode_tps = -n / dt
            for seq_id, toks in outputs:
                done[seq_id] = toks
            if use_tqdm and perf_counter() - last_print > 1.0:
                last_print = perf_counter()
                print(f"\rGenerating: {len(done)}/{len(ids)}  Prefill {int(prefill_tps)} tok/s  "
                      f"Decode {int(decode_tps)} tok/s", end="", file=sys.stderr, flush=True)
        if use_tqdm:
            print(f"\rGenerating: {len(done)}/{len(ids)} done" + " " * 40, file=sys.stderr, flush=True)
        self.model.kernels.check_faults()
        results = []
        for seq_id in ids:
            toks = done[seq_id]
            seq = self._by_id.pop(seq_id)
            text = None
            if self.tokenizer is not None:
                text = self.tokenizer.decode(toks)
            results.append({"text": text, "token_ids": toks, "finish_reason": seq.finish_reason})
        return results

    def exit(self):
        pass
