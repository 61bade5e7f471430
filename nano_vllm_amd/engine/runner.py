"""The model runner: owns the model, the cache tensors and the step function.

Reference: nanovllm/engine/model_runner.py - ModelRunner.run (:214-220) with its
prepare_* helpers, allocate_kv_cache (:103-121).  One step function serves every caller
(the engine loop and the trace replay): it runs exactly the tokens it is given, as one
batch, from the cache, and returns float32 logits at the wanted places.  Sampling is a
separate call.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..cache.manager import CacheManager, plan_groups
from ..cache.pages import OutOfPages
from ..cache import storage
from ..config.model_config import read_config_json
from ..config.registry import architecture_of
from ..kernels import HipKernels
from ..parts.model import Model, torch_dtype
from ..weights.loader import load_weights
from ..weights.random_weights import fill_random_
from .batch import StepEntry, build_batch


class ModelRunner:
    def __init__(self, model: Model, page_size: int, num_pages, max_requests: int,
                 enable_prefix_caching: bool = True):
        """num_pages: pages per cache group (an int for every group, or one per group)."""
        self.model = model
        self.kernels = model.kernels
        self.device = model.device
        self.page_size = page_size
        self.needs = model.cache_needs()
        self.groups, self.state_runs = plan_groups(self.needs)
        counts = list(num_pages) if isinstance(num_pages, (list, tuple)) else [num_pages] * len(self.groups)
        self.cache = CacheManager(self.groups, page_size, counts,
                                  num_state_slots=max_requests if self.state_runs else 0,
                                  has_state=bool(self.state_runs), enable_prefix_caching=enable_prefix_caching)
        self.layer_caches = storage.allocate(self.needs, self.groups, self.state_runs, counts, page_size,
                                             max_requests, model.dtype, self.device)
        self._graphs = {}
        self._graph_pool = None
        self._graph_max_batch = 0
        self._graph_max_len = 0

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_folder(cls, folder: str, dtype: Optional[str] = None, device="cuda:0", page_size: int = 256,
                    num_pages=None, max_requests: int = 512, kernels=None, quiet: bool = False,
                    enable_prefix_caching: bool = True) -> "ModelRunner":
        model = load_model(folder, dtype, device, kernels, quiet)
        return cls(model, page_size, num_pages, max_requests, enable_prefix_caching)

    # ------------------------------------------------------------------ the step
    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Runs the entries' tokens as one batch.  Their pages must be reserved in
        self.cache.  Returns float32 logits [wanted places, vocab] in the order of the
        entries and of their `want`, or None if nothing is wanted.  (With decode graphs
        enabled the tensor returned for a pure decode step is overwritten by the next such
        step of the same batch size.)"""
        if self._graph_max_batch and self._graph_takes(entries):
            return self._step_graph(entries)
        batch = build_batch(entries, self.cache, self.page_size, self.model.spec.vocab_size, self.device,
                            max_position=self.model.spec.max_position,
                            extras=getattr(self.kernels, "batch_extras", None))
        hidden = self.model.forward(batch, self.layer_caches)
        if batch.logits_rows is None:
            return None
        return self.model.logits(hidden, batch.logits_rows)

    # ------------------------------------------------------------------ captured decode steps
    def enable_decode_graphs(self, max_batch: int, max_len: int, measure_products: bool = True) -> None:
        """Decode steps (one token per request, its logits wanted) of up to max_batch requests
        and max_len cached tokens are captured as HIP graphs, one per padded batch size, at
        their first occurrence, and replayed from then on.  Reference: capture_cudagraph and
        the replay branch of run_model (nanovllm/engine/model_runner.py:195-212,222-257),
        which captures every size at start-up."""
        if any(not self.model.blocks[self.model.order[i].layer].replays_state_steps for i in self.state_runs):
            return          # a mixer that handles its state on the host cannot be replayed blindly
        if max_len > self.model.spec.max_position:
            raise ValueError(f"decode graphs for {max_len} tokens: the model knows {self.model.spec.max_position} positions")
        # which product kernel serves which row count of these steps: measured on the model's own
        # weights, unless a record of an earlier measurement exists (or the caller wants the rules alone)
        if measure_products and self.device.type == "cuda" and hasattr(self.kernels, "choose_products"):
            self.kernels.choose_products(self.model.params.values(), max_batch)
        self._graph_max_batch = max_batch
        self._graph_max_len = max_len
        self._graph_table_width = (max_len + self.page_size - 1) // self.page_size

    @torch.inference_mode()          # as step(): every capture of a process happens in the same mode
    def capture_decode_graphs(self) -> int:
        """Captures every batch size now, the largest first (so that the smaller ones find their
        memory in the shared pool), with stand-in requests of one token each; what cannot be
        captured for want of pages or request slots is left for its first occurrence.  Returns the
        number of sizes captured.  (nanovllm/engine/model_runner.py:222-257 does this at start-up.)"""
        if not self._graph_max_batch or self.device.type != "cuda":
            return 0
        sizes = sorted({self.graph_batch_size(n) for n in range(1, self._graph_max_batch + 1)}, reverse=True)
        done = 0
        for b in sizes:
            if b in self._graphs or b > self._graph_max_batch or any(pool.num_free < b for pool in self.cache.pools) \
                    or (self.cache.slots.num_slots and self.cache.slots.num_free < b):
                continue
            names = [("captured decode step", i) for i in range(b)]
            held = []
            try:
                for name in names:
                    self.cache.admit(name)
                    held.append(name)
                    self.cache.reserve(name, 1)
                self._step_graph([StepEntry(name, [0], 0, [0]) for name in names])
                done += 1
            except OutOfPages:
                pass
            finally:
                for name in held:
                    self.cache.release(name)
        return done

    def _graph_takes(self, entries) -> bool:
        if len(entries) > self._graph_max_batch or self.device.type != "cuda":
            return False
        for e in entries:
            if len(e.tokens) != 1 or len(e.want) != 1 or e.want[0] != 0 or e.start + 1 > self._graph_max_len:
                return False
        return True

    @staticmethod
    def graph_batch_size(n: int) -> int:
        """The captured batch size that serves n requests: 1, 2, 4, 8, then multiples of 16
        (the reference's buckets, nanovllm/engine/model_runner.py:226)."""
        for b in (1, 2, 4, 8):
            if n <= b:
                return b
        return (n + 15) // 16 * 16

    def _step_graph(self, entries) -> torch.Tensor:
        n = len(entries)
        size_b = self.graph_batch_size(n)
        vocab = self.model.spec.vocab_size
        g = self._graphs.get(size_b)
        if g is None:
            # the flat layout of size_b single tokens with every logit wanted and tables of fixed width
            num_groups = len(self.groups)
            b = size_b
            size = 3 * b + (b + 1) + 3 * b + b + num_groups * (b + b * self._graph_table_width)
            static = torch.zeros(size, dtype=torch.int32, device=self.device)
            batch = build_batch(entries, self.cache, self.page_size, vocab, self.device,
                                table_width=self._graph_table_width, static=static, pad_to=size_b,
                                max_position=self.model.spec.max_position)
            batch.max_kv_len = self._graph_max_len        # launch shapes must cover every later step
            # The set-up runs below are real steps of these requests.  For keys and values that is
            # harmless (the replay writes the same numbers to the same slots again); per-request
            # state would be advanced three times, so the rows of this batch are put back afterwards.
            rows = batch.state_slots.long() if self.state_runs else None
            saved = [{name: t.index_select(0, rows) for name, t in self.layer_caches[i].state.items()}
                     for i in self.state_runs]
            side = torch.cuda.Stream(self.device)
            side.wait_stream(torch.cuda.current_stream(self.device))
            with torch.cuda.stream(side):                 # what is set up lazily is set up outside the capture
                for _ in range(2):
                    self.model.logits(self.model.forward(batch, self.layer_caches), batch.logits_rows)
            torch.cuda.current_stream(self.device).wait_stream(side)
            torch.cuda.synchronize(self.device)
            for i, kept in zip(self.state_runs, saved):
                for name, t in kept.items():
                    self.layer_caches[i].state[name].index_copy_(0, rows, t)
            graph = torch.cuda.CUDAGraph()
            if self._graph_pool is None:                  # one memory pool for all sizes: they run one at a time
                self._graph_pool = torch.cuda.graph_pool_handle()
            with torch.cuda.graph(graph, pool=self._graph_pool):
                logits = self.model.logits(self.model.forward(batch, self.layer_caches), batch.logits_rows)
            g = (graph, static, logits, batch)
            self._graphs[size_b] = g
        graph, static, logits, _ = g
        build_batch(entries, self.cache, self.page_size, vocab, self.device,
                    table_width=self._graph_table_width, static=static, pad_to=size_b,
                    max_position=self.model.spec.max_position)
        graph.replay()
        return logits[:n]

    @torch.inference_mode()
    def decode_burst(self, entries: Sequence[StepEntry], steps: int, sampler, temperatures, seeds,
                     requests) -> List[List[int]]:
        """`steps` decode steps of the same requests without the host in between: after each
        captured step the tokens are sampled on the device and a small kernel writes the next
        step's metadata (tokens, positions, slots) in place.  The entries are the first step's;
        pages for the positions of all the steps must be reserved.  Returns the sampled tokens,
        [steps][requests]; they are exactly those of `steps` single steps.  (The reference
        returns to the host after every step, nanovllm/engine/llm_engine.py:49-55.)"""
        n = len(entries)
        if not (self._graph_max_batch and self._graph_takes(entries)):
            raise ValueError("decode_burst needs captured decode steps and a batch they take")
        if any(e.start + steps > self._graph_max_len for e in entries):
            raise ValueError("decode_burst: the steps run past the captured length")
        self._step_graph(entries)
        graph, _, logits, batch = self._graphs[self.graph_batch_size(n)]
        positions = [[e.start + 1 + j for e in entries] for j in range(steps)]
        temps, keys = sampler.device_inputs(temperatures, seeds, requests, positions)
        out = torch.empty((steps, n), dtype=torch.int32, device=self.device)
        kernels = self.model.kernels
        for j in range(steps):
            ids = kernels.sample(logits[:n], temps, keys[j])
            if j + 1 < steps:
                kernels.advance_decode(batch, ids, out[j], n, self.page_size)
                graph.replay()
            else:
                out[j].copy_(ids)
        return out.tolist()


def load_model(folder: str, dtype: Optional[str] = None, device="cuda:0", kernels=None, quiet: bool = False,
               random_weights: Optional[int] = None) -> Model:
    """config.json -> architecture -> ModelSpec -> Model, then the weights of the folder, or,
    with a seed in random_weights, random weights drawn on the device."""
    config_json = read_config_json(folder)
    arch = architecture_of(config_json)
    config = arch.parse_config(config_json)
    spec = arch.build_spec(config)
    tdtype = torch_dtype(dtype or spec.dtype)
    if kernels is None:
        kernels = HipKernels(device, tdtype, quiet=quiet)        # raises without a GPU or the compiled kernels
    model = Model(spec, kernels, device, tdtype)
    if random_weights is None:
        load_weights(model, folder)
    else:
        fill_random_(model, random_weights)
    return model
