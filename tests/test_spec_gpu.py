"""The model as data: an execution order that names a layer twice and lets a layer read
another layer's cache, layers with a window beside layers that keep every key (two cache
groups, pages of the window group given back while a request runs), and the layer sizes of
the Qwen3-8B shape - each driven through the step function in portions and compared with
the plain implementation."""
import dataclasses
import json
import os

import pytest
import torch

import helpers as H
import plain_qwen3 as plain
from nano_vllm_amd.config import Qwen3Config, register_architecture
from nano_vllm_amd.engine.batch import StepEntry
from nano_vllm_amd.engine.runner import ModelRunner
from nano_vllm_amd.models.qwen3 import build_spec
from nano_vllm_amd.parts import LayerRun, PartSpec
from nano_vllm_amd.weights import write_random_model

pytestmark = pytest.mark.gpu

ORDER = [(0, None), (1, None), (1, None), (2, 0)]       # layer 1 runs twice; the last run reads the first run's cache
WINDOWS = {1: 12}


def _variant_spec(cfg: Qwen3Config):
    """Qwen3's parts with another arrangement: layer 1 has a window, layer 2 projects q only."""
    spec = build_spec(cfg)
    layers = list(spec.layers)

    def with_mixer(layer, **kw):
        parts = dict(layer.parts)
        parts["mixer"] = PartSpec("attention", {**parts["mixer"].params, **kw})
        return dataclasses.replace(layer, parts=parts)

    layers[1] = with_mixer(layers[1], window=WINDOWS[1])
    layers[2] = with_mixer(layers[2], reads_shared_cache=True)
    order = tuple(LayerRun(layer, source) for layer, source in ORDER)
    return dataclasses.replace(spec, architecture="Qwen3VariantForTest", layers=tuple(layers), order=order)


def _parse(d):
    return Qwen3Config.from_dict({**d, "architectures": ["Qwen3ForCausalLM"]})


@pytest.fixture(scope="module")
def variant_folder(tmp_path_factory):
    register_architecture("Qwen3VariantForTest", _parse, _variant_spec, replace=True)
    cfg = H.CONFIGS["b"]["cfg"]
    folders = {}
    for dtype in ("float32", "bfloat16"):
        cj = cfg.to_dict()
        cj["architectures"] = ["Qwen3VariantForTest"]
        folders[dtype] = write_random_model(str(tmp_path_factory.mktemp("variant") / dtype), cj, seed=21, norm_std=0.1,
                                            dtype=dtype)
    return folders


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_order_shared_cache_and_window_groups(variant_folder, dtype):
    folder = variant_folder[dtype]
    r = ModelRunner.from_folder(folder, dtype=dtype, page_size=8, num_pages=[56, 16], max_requests=4, quiet=True,
                                enable_prefix_caching=False)
    assert [(g.window, g.runs) for g in r.groups] == [(None, (0,)), (12, (1, 2))]
    assert r.needs[3] is None and r.model.cache_owner(3) == 0
    assert "model.layers.2.self_attn.k_proj.weight" not in json.dumps(sorted(r.model.params))
    assert r.model.params["model.layers.2.self_attn.qkv_proj.weight"].shape[0] == 8 * 32      # q rows only
    cfg, w = plain.read_folder(folder)
    rounding = None if dtype == "float32" else "bfloat16"
    tol = 2e-5 if dtype == "float32" else 2e-2
    reqs = {f"r{i}": H.random_tokens(cfg.vocab_size, n, 90 + i) for i, n in enumerate((150, 97, 61, 120))}
    want = {k: plain.logits(w, cfg, v, rounding, order=ORDER, windows=WINDOWS) for k, v in reqs.items()}
    # alone, in portions of changing size
    got = H.run_portions(r, "x", reqs["r0"], H.changing_portions(150, 3))
    assert H.rel_err(got, want["r0"]) < tol
    # the window group holds 16 pages of 8 where the four requests have 55 pages of tokens: they
    # only fit because pages that the window has passed are given back while the requests run
    got = H.run_mixed_groups(r, reqs, seed=6)
    for k in reqs:
        assert H.rel_err(got[k], want[k]) < tol, k
    assert r.cache.pools[0].num_free == 56 and r.cache.pools[1].num_free == 16
    r.kernels.check_faults()


@pytest.fixture(scope="module")
def real_size_folder(tmp_path_factory):
    """name -> folder of two layers with the layer sizes of a named Qwen3 shape (a smaller vocabulary
    keeps the plain implementation quick), weights stored in bfloat16: the float32 engine and the
    plain implementation widen the same numbers, so one folder serves both element types."""
    from nano_vllm_amd.models.shapes import shape
    folders = {}

    def get(name):
        if name not in folders:
            cj = shape(name)
            cj.update(num_hidden_layers=2, vocab_size=2048, max_position_embeddings=4096)
            folders[name] = write_random_model(str(tmp_path_factory.mktemp(name) / "m"), cj, seed=5, dtype="bfloat16")
        return folders[name]
    return get


# 8B: 32 heads in groups of four; 14B: 40 heads in groups of five, widths of 5120 and 17408;
# 32B: 64 heads in groups of eight, 25600 inner channels: other instances of the product and
# attention kernels than the 8B sizes run.  0.6B, 1.7B, 4B: groups of two, q heads wider than the
# model (2048 of 1024), widths of 2560 and 9728, a tied head.
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["qwen3-0.6b", "qwen3-1.7b", "qwen3-4b", "qwen3-8b", "qwen3-14b", "qwen3-32b"])
def test_layer_sizes_of_the_named_shapes(real_size_folder, name, dtype):
    """Two layers with the layer sizes of the benchmarks' shapes: float32 against the plain
    implementation, whole, decoded and in portions; bfloat16 against the plain implementation with
    bfloat16 roundings; then several requests in one step on a short pool."""
    folder = real_size_folder(name)
    r = ModelRunner.from_folder(folder, dtype=dtype, page_size=256, num_pages=4, max_requests=2, quiet=True,
                                enable_prefix_caching=False)
    if dtype == "bfloat16":
        # what an engine does at start-up: the product kernels for 17 to 256 rows are the ones the
        # model's own weights choose, and those are the ones compared below
        r.kernels.choose_products(r.model.params.values(), 256)
    n = 300                                   # crosses a page of 256
    toks = H.random_tokens(2048, n, 7)
    pcfg, w = plain.read_folder(folder)
    rounding = None if dtype == "float32" else "bfloat16"
    want = plain.logits(w, pcfg, toks, rounding)
    tol = 2e-5 if dtype == "float32" else 2e-2
    # 41, 100, 200, 241 rows: the kernels for medium row counts
    for portions in ([n], [n - 32] + [1] * 32, [250, 2, 7, 41], [100, 200], [59, 241]):
        got = H.run_portions(r, "x", toks, portions)
        assert H.rel_err(got, want) < tol, portions
    r.kernels.check_faults()
    # several requests in one step at these sizes: single tokens of three beside a portion of a
    # fourth, pages of 256, on a pool that holds three of the five requests
    lens = [300, 270, 40, 290, 180]
    reqs = {f"r{i}": H.random_tokens(2048, m, 20 + i) for i, m in enumerate(lens)}
    choice = dict(getattr(r.kernels, "product_choice", {}))
    del r
    r = ModelRunner.from_folder(folder, dtype=dtype, page_size=256, num_pages=5, max_requests=4, quiet=True,
                                enable_prefix_caching=False)
    if dtype == "bfloat16":
        r.kernels.product_choice = choice
    got = H.run_mixed(r, reqs, seed=9)
    for rid, t in reqs.items():
        assert H.rel_err(got[rid], plain.logits(w, pcfg, t, rounding)) < tol, rid
    assert r.cache.pools[0].num_free == 5
    r.kernels.check_faults()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_that_lie_beyond_four_gibibytes_of_a_layers_keys(real_size_folder, dtype):
    """A cache as large as a serving engine's: pages of 256 tokens of the 8B shape's 8 kv heads of
    128 are 512 KiB of a layer's keys each (1 MiB in float32), so page 8192 begins 2^31 elements and
    4 GiB (8 GiB) into the tensor.  With the first 8200 pages held by another request, a request's pages lie beyond
    that: its keys and values are written there, by a prompt's portions and by single tokens, and
    read from there, and the logits are those of the plain implementation."""
    folder = real_size_folder("qwen3-8b")
    first = 8200
    r = ModelRunner.from_folder(folder, dtype=dtype, page_size=256, num_pages=first + 6, max_requests=4, quiet=True,
                                enable_prefix_caching=False)
    pool = r.cache.pools[0]
    r.cache.admit("holds the first pages")
    r.cache.reserve("holds the first pages", first * 256)
    assert sorted(r.cache.table("holds the first pages", 0)) == list(range(first))
    toks = H.random_tokens(2048, 300, 7)
    pcfg, w = plain.read_folder(folder)
    want = plain.logits(w, pcfg, toks, None if dtype == "float32" else "bfloat16")
    tol = 2e-5 if dtype == "float32" else 2e-2
    for portions in ([300 - 32] + [1] * 32, [250, 2, 7, 41]):
        r.cache.admit("x")
        out, pos = [], 0
        for n in portions:
            r.cache.reserve("x", pos + n)
            assert min(r.cache.table("x", 0)) >= first
            out.append(r.step([StepEntry("x", toks[pos:pos + n], pos, list(range(n)))]).float().cpu())
            pos += n
        r.cache.release("x")
        assert H.rel_err(torch.cat(out), want) < tol, portions
    # two requests in one step: single tokens of one beside a portion of the other
    reqs = {"a": H.random_tokens(2048, 290, 21), "b": H.random_tokens(2048, 270, 22)}
    got = H.run_mixed(r, reqs, seed=4)
    for rid, t in reqs.items():
        assert H.rel_err(got[rid], plain.logits(w, pcfg, t, None if dtype == "float32" else "bfloat16")) < tol, rid
    r.kernels.check_faults()
    r.cache.release("holds the first pages")
    r.cache.check()
    assert pool.num_free == first + 6


def test_two_engines_on_one_model_choose_the_same_product_kernels(real_size_folder, tmp_path, monkeypatch):
    """The product kernels for 17 to 256 rows are measured once and recorded: a second engine, and
    a second process (its table emptied here, so that it comes from the record), run the same
    kernels and give the same bfloat16 logits bit for bit at 17, 64 and 240 rows."""
    from nano_vllm_amd.kernels import ops
    record = tmp_path / "product_choice.json"
    monkeypatch.setattr(ops, "_choice_file", lambda write=False: str(record) if write or record.exists() else None)
    monkeypatch.setattr(ops, "_product_choices", {})
    folder = real_size_folder("qwen3-8b")
    toks = H.random_tokens(2048, 17 + 64 + 240, 31)

    def logits_of_an_engine():
        r = ModelRunner.from_folder(folder, dtype="bfloat16", page_size=256, num_pages=4, max_requests=2, quiet=True,
                                    enable_prefix_caching=False)
        r.enable_decode_graphs(256, 2048)           # measures, or finds the record
        table = {key: dict(rows) for key, rows in r.kernels.product_choice.items()}
        return H.run_portions(r, "x", toks, [17, 64, 240]), table

    first, table = logits_of_an_engine()
    assert record.exists() and (4096, 12288, False) in table and (24576, 4096, True) in table
    assert all(set(rows) == set(range(2, 17)) for rows in table.values())
    second, table2 = logits_of_an_engine()
    monkeypatch.setattr(ops, "_product_choices", {})      # as in a new process
    third, table3 = logits_of_an_engine()
    assert table2 == table and table3 == table
    assert torch.equal(first, second) and torch.equal(first, third)


def test_the_cache_is_sized_from_the_measured_peak_of_the_largest_step(real_size_folder):
    """nanovllm/engine/model_runner.py:91-114: the largest step is run once before the cache is
    sized.  With 12 GiB granted beyond what is in use, a step of 16384 prompt tokens through the
    engine stays inside the grant, and the grant is used: pages, weights and the measured peak fill it."""
    from nano_vllm_amd import LLM, SamplingParams
    folder = real_size_folder("qwen3-8b")
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    free, total = torch.cuda.mem_get_info()
    in_use = total - free                         # other processes, and what earlier tests still hold
    held_here = torch.cuda.memory_allocated()
    grant = 12 << 30
    llm = LLM(folder, dtype="bfloat16", gpu_memory_utilization=(in_use + grant) / total, max_num_batched_tokens=16384,
              max_model_len=4096, max_num_seqs=8, enable_prefix_caching=False)
    per_page = 2 * 2 * 8 * 128 * 256 * 2          # K and V, two layers, 8 kv heads of 128, pages of 256, bfloat16
    cache_bytes = llm.config.num_kvcache_blocks * per_page
    weights = sum(t.numel() * t.element_size() for t in llm.model.params.values())
    assert llm.warmup_peak_bytes > 16384 * 4096 * 2 * 4       # a few rows of the width per token at the least
    # (what is in use is read before and after the model is loaded: the two readings differ by what the
    # allocator and the libraries hold in between, tens of MiB)
    assert grant - (256 << 20) <= cache_bytes + weights + llm.warmup_peak_bytes + 15 * 2048 * 4 <= grant + (64 << 20)
    torch.cuda.reset_peak_memory_stats()
    prompts = [H.random_tokens(2048, 4094, 50 + i) for i in range(4)] + [H.random_tokens(2048, 8, 60)]
    outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=2), use_tqdm=False)
    assert [len(o["token_ids"]) for o in outs] == [2] * 5 and llm.stats["steps"] <= 4      # all prompts in one step
    assert torch.cuda.max_memory_allocated() - held_here <= grant + (64 << 20)
