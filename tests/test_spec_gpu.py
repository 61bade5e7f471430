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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layer_sizes_of_the_8b_shape(tmp_path, dtype):
    """Two layers with the Qwen3-8B layer sizes (a smaller vocabulary keeps the plain
    implementation quick): float32 against the plain implementation, whole, decoded and in
    portions; bfloat16 against the plain implementation with bfloat16 roundings."""
    cfg = Qwen3Config(vocab_size=2048, hidden_size=4096, num_hidden_layers=2, num_attention_heads=32,
                      num_key_value_heads=8, head_dim=128, intermediate_size=12288, rms_norm_eps=1e-6,
                      rope_theta=1000000.0, max_position_embeddings=4096, tie_word_embeddings=False)
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=5, dtype=dtype)
    r = ModelRunner.from_folder(folder, dtype=dtype, page_size=256, num_pages=4, max_requests=2, quiet=True,
                                enable_prefix_caching=False)
    n = 300                                   # crosses a page of 256
    toks = H.random_tokens(2048, n, 7)
    pcfg, w = plain.read_folder(folder)
    want = plain.logits(w, pcfg, toks, None if dtype == "float32" else "bfloat16")
    tol = 2e-5 if dtype == "float32" else 2e-2
    for portions in ([n], [n - 32] + [1] * 32, [250, 2, 7, 41], [100, 200]):       # 41, 100, 200 rows: the kernel for medium row counts
        got = H.run_portions(r, "x", toks, portions)
        assert H.rel_err(got, want) < tol, portions
    r.kernels.check_faults()
    del r
    # several requests in one step at these sizes: single tokens of three beside a portion of a
    # fourth, pages of 256, on a pool that holds three of the five requests
    lens = [300, 270, 40, 290, 180]
    reqs = {f"r{i}": H.random_tokens(2048, m, 20 + i) for i, m in enumerate(lens)}
    r = ModelRunner.from_folder(folder, dtype=dtype, page_size=256, num_pages=5, max_requests=4, quiet=True,
                                enable_prefix_caching=False)
    got = H.run_mixed(r, reqs, seed=9)
    for rid, t in reqs.items():
        want = plain.logits(w, pcfg, t, None if dtype == "float32" else "bfloat16")
        assert H.rel_err(got[rid], want) < tol, rid
    assert r.cache.pools[0].num_free == 5
    r.kernels.check_faults()
