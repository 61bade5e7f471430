"""The engine on a model with two cache groups (layers that keep every key beside a layer with a
window): LLM.generate under both schedules, with prompts cut into portions of 2, 5 and 16 tokens
and a window pool so small that pages the window has passed must be given back while prompts are
still being cut and while requests decode.  The tokens are the plain implementation's; the cache
manager's books balance afterwards.  Then with prefix reuse: requests that begin like an earlier one
leave out the pages that both groups still stand for.  Once on the CPU stand-ins of the kernels,
once on the GPU."""
import dataclasses

import pytest
import torch

import helpers as H
import plain_qwen3 as plain
from nano_vllm_amd import LLM, SamplingParams
from nano_vllm_amd.config import Qwen3Config, register_architecture
from nano_vllm_amd.models.qwen3 import build_spec
from nano_vllm_amd.parts import LayerRun, PartSpec
from nano_vllm_amd.weights import write_random_model
from torch_kernels import TorchKernels

ORDER = [(0, None), (1, None), (2, None)]
WINDOWS = {1: 12}
PAGE = 8


def _spec(cfg: Qwen3Config):
    spec = build_spec(cfg)
    layers = list(spec.layers)
    parts = dict(layers[1].parts)
    parts["mixer"] = PartSpec("attention", {**parts["mixer"].params, "window": WINDOWS[1]})
    layers[1] = dataclasses.replace(layers[1], parts=parts)
    return dataclasses.replace(spec, architecture="Qwen3WindowForTest", layers=tuple(layers))


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    register_architecture("Qwen3WindowForTest", lambda d: Qwen3Config.from_dict({**d, "architectures": ["Qwen3ForCausalLM"]}),
                          _spec, replace=True)
    cj = H.CONFIGS["b"]["cfg"].to_dict()
    cj["architectures"] = ["Qwen3WindowForTest"]
    return write_random_model(str(tmp_path_factory.mktemp("window") / "m"), cj, seed=23, norm_std=0.1, dtype="float32")


@pytest.fixture(scope="module")
def expected(folder):
    cfg, w = plain.read_folder(folder)
    prompts = [H.random_tokens(cfg.vocab_size, n, 300 + n) for n in (37, 61, 5, 50, 26)]
    want = []
    for p in prompts:
        ids = list(p)
        for _ in range(10):          # ten tokens: every request decodes across the window's edge and a page's
            ids.append(int(torch.argmax(plain.logits(w, cfg, ids, None, order=ORDER, windows=WINDOWS)[-1])))
        want.append(ids[len(p):])
    return prompts, want


def _generate(folder, expected, schedule, budget, window_pages, **where):
    prompts, want = expected
    llm = LLM(folder, dtype="float32", kvcache_block_size=PAGE, num_kvcache_blocks=[40, window_pages],
              max_num_batched_tokens=budget, max_num_seqs=3, schedule=schedule, enable_prefix_caching=False, **where)
    cache = llm.runner.cache
    assert [g.window for g in cache.groups] == [None, WINDOWS[1]]
    # no more than a request holds at its peak, and less than the prompts' own pages: 61 tokens are 8 pages
    peak = cache.peak_pages(71, budget)[1]
    assert window_pages <= peak + 2 and peak < 8
    low = [window_pages]
    step = llm.step

    def watched_step():
        out = step()
        cache.check()
        low[0] = min(low[0], cache.pools[1].num_free)
        return out
    llm.step = watched_step
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10), use_tqdm=False)
    assert [o["token_ids"] for o in outs] == want, (schedule, budget)
    assert all(o["finish_reason"] == "max_tokens" for o in outs)
    assert cache.pools[0].num_free == 40 and cache.pools[1].num_free == window_pages and not cache.requests
    assert low[0] <= 1, "the window pool was never short: the test shows nothing"
    return llm


@pytest.mark.parametrize("schedule", ["prefill_first", "mixed"])
@pytest.mark.parametrize("budget", [2, 5, 16])
def test_window_group_through_the_engine_on_cpu_stand_ins(folder, expected, schedule, budget):
    pages = {2: 4, 5: 4, 16: 5}[budget]
    _generate(folder, expected, schedule, budget, pages, kernels=TorchKernels(), device="cpu")


@pytest.mark.gpu
@pytest.mark.parametrize("schedule", ["prefill_first", "mixed"])
@pytest.mark.parametrize("budget", [2, 5, 16])
def test_window_group_through_the_engine(folder, expected, schedule, budget):
    pages = {2: 4, 5: 4, 16: 5}[budget]
    llm = _generate(folder, expected, schedule, budget, pages)
    llm.model.kernels.check_faults()


# ------------------------------------------------------------------------------ prefix reuse over both groups
def _plain_tokens(folder, prompt, n=10):
    cfg, w = plain.read_folder(folder)
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(torch.argmax(plain.logits(w, cfg, ids, None, order=ORDER, windows=WINDOWS)[-1])))
    return ids[len(prompt):]


def _reuse(folder, window_pages, **where):
    """One request, then two that begin with its first 43 tokens (five pages and three tokens) and
    one that does not.  With a window pool that keeps the first request's pages, the two leave out
    40 tokens each: the all-keys group stands for five pages, the window group for the two that
    position 40 looks back at (window 12: positions 29..39, pages 3 and 4)."""
    V = H.CONFIGS["b"]["cfg"].vocab_size
    stem = H.random_tokens(V, 43, 700)
    first = stem + H.random_tokens(V, 9, 701)
    later = [stem + H.random_tokens(V, 14, 702), H.random_tokens(V, 30, 703), stem + H.random_tokens(V, 3, 704)]
    llm = LLM(folder, dtype="float32", kvcache_block_size=PAGE, num_kvcache_blocks=[40, window_pages],
              max_num_batched_tokens=16, max_num_seqs=3, **where)
    cache = llm.runner.cache
    assert cache.prefix_caching
    step = llm.step

    def watched_step():
        out = step()
        cache.check()
        return out
    llm.step = watched_step
    sp = SamplingParams(temperature=0.0, max_tokens=10)
    out = llm.generate([first], sp, use_tqdm=False)
    assert out[0]["token_ids"] == _plain_tokens(folder, first)
    assert llm.stats["prefill_tokens"] == len(first)
    outs = llm.generate(later, sp, use_tqdm=False)
    assert [o["token_ids"] for o in outs] == [_plain_tokens(folder, p) for p in later]
    assert cache.pools[0].num_free == 40 and cache.pools[1].num_free == window_pages and not cache.requests
    return llm.stats["prefill_tokens"] - len(first), sum(len(p) for p in later)


@pytest.mark.parametrize("window_pages", [12, 5])
def test_prefix_reuse_with_a_window_group_on_cpu_stand_ins(folder, window_pages):
    computed, asked = _reuse(folder, window_pages, kernels=TorchKernels(), device="cpu")
    if window_pages == 12:
        assert computed == asked - 2 * 40         # both later requests with the stem leave out five pages
    else:
        assert computed <= asked                  # the window's pages were taken again: less is left out, or nothing


@pytest.mark.gpu
@pytest.mark.parametrize("window_pages", [12, 5])
def test_prefix_reuse_with_a_window_group(folder, window_pages):
    computed, asked = _reuse(folder, window_pages)
    assert computed == asked - 2 * 40 if window_pages == 12 else computed <= asked
