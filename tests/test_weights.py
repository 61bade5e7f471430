"""Weights: names, packing, element types, the one error that lists everything, and the
random-weights mode's model folder."""
import json
import os

import pytest
import torch
from safetensors import safe_open
from safetensors.torch import load_file, save_file

from nano_vllm_amd.engine.runner import load_model
from nano_vllm_amd.weights import WeightError, random_checkpoint, write_random_model

from helpers import CONFIGS
from torch_kernels import TorchKernels


def _load(folder, dtype=None):
    return load_model(folder, dtype, "cpu", kernels=TorchKernels())


def _folder(tmp_path, name="b", dtype="float32", **kw):
    c = CONFIGS[name]
    return write_random_model(str(tmp_path / f"{name}-{dtype}"), c["cfg"], seed=c["seed"], norm_std=c["norm_std"],
                              dtype=dtype, **kw)


def test_folder_has_checkpoint_names_and_shapes(tmp_path):
    folder = _folder(tmp_path, "b")
    cfg = CONFIGS["b"]["cfg"]
    with open(os.path.join(folder, "config.json")) as f:
        cj = json.load(f)
    assert cj["architectures"] == ["Qwen3ForCausalLM"] and cj["hidden_size"] == cfg.hidden_size
    t = load_file(os.path.join(folder, "model.safetensors"))
    D, H = cfg.head_dim, cfg.hidden_size
    assert t["model.layers.2.self_attn.q_proj.weight"].shape == (cfg.num_attention_heads * D, H)
    assert t["model.layers.2.self_attn.k_proj.weight"].shape == (cfg.num_key_value_heads * D, H)
    assert t["model.layers.0.self_attn.q_norm.weight"].shape == (D,)
    assert t["model.layers.1.mlp.up_proj.weight"].shape == (cfg.intermediate_size, H)
    assert t["lm_head.weight"].shape == (cfg.vocab_size, H) and t["model.norm.weight"].shape == (H,)
    assert len(t) == 3 + 11 * cfg.num_hidden_layers
    assert not any("qkv_proj" in n or "gate_up" in n or "rotary" in n for n in t)


def test_tied_folder_holds_no_head(tmp_path):
    folder = _folder(tmp_path, "a")
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        assert "lm_head.weight" not in f.keys()
    m = _load(folder)
    assert m.head.weights["weight"] is m.embedding.weights["weight"]


def test_seed_decides_the_values(tmp_path):
    cj = CONFIGS["a"]["cfg"].to_dict()
    a, b, c = random_checkpoint(cj, 1), random_checkpoint(cj, 1), random_checkpoint(cj, 2)
    assert all(torch.equal(a[n], b[n]) for n in a)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    assert abs(float(a["model.embed_tokens.weight"].float().std()) - 0.02) < 0.002
    assert torch.equal(a["model.norm.weight"].float(), torch.ones(64))


def test_packed_parameters_are_the_concatenation(tmp_path):
    folder = _folder(tmp_path, "b")
    t = load_file(os.path.join(folder, "model.safetensors"))
    m = _load(folder)
    p = "model.layers.1"
    qkv = torch.cat([t[f"{p}.self_attn.{n}_proj.weight"] for n in "qkv"])
    assert torch.equal(m.params[f"{p}.self_attn.qkv_proj.weight"], qkv)
    gu = torch.cat([t[f"{p}.mlp.gate_proj.weight"], t[f"{p}.mlp.up_proj.weight"]])
    assert torch.equal(m.params[f"{p}.mlp.gate_up_proj.weight"], gu)
    assert torch.equal(m.params[f"{p}.mlp.down_proj.weight"], t[f"{p}.mlp.down_proj.weight"])


def test_element_types(tmp_path):
    f32 = _folder(tmp_path, "b", "float32")
    bf = _folder(tmp_path, "b", "bfloat16")
    m = _load(bf)                                     # config.json says bfloat16
    assert m.dtype == torch.bfloat16 and all(p.dtype == torch.bfloat16 for p in m.params.values())
    m = _load(bf, "float32")                          # widened exactly
    assert all(p.dtype == torch.float32 for p in m.params.values())
    t = load_file(os.path.join(bf, "model.safetensors"))
    assert torch.equal(m.params["model.norm.weight"], t["model.norm.weight"].float())
    m = _load(f32, "bfloat16")
    # matrices are kept in bfloat16; a vector stored in 32 bits stays so
    assert m.params["model.layers.0.mlp.down_proj.weight"].dtype == torch.bfloat16
    assert m.params["model.embed_tokens.weight"].dtype == torch.bfloat16
    assert m.params["model.norm.weight"].dtype == torch.float32
    assert m.params["model.layers.0.self_attn.q_norm.weight"].dtype == torch.float32


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = _folder(tmp_path, "b")
    path = os.path.join(folder, "model.safetensors")
    t = load_file(path)
    del t["model.layers.0.self_attn.k_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    t["model.layers.9.mlp.up_proj.weight"] = torch.zeros(2, 2)
    t["model.layers.1.mlp.down_proj.weight"] = torch.zeros(96, 161)
    t["model.layers.2.self_attn.q_norm.weight"] = torch.zeros(31)
    save_file(t, path)
    with pytest.raises(WeightError) as e:
        _load(folder)
    err = e.value
    assert err.missing == ["model.layers.0.self_attn.k_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq", "model.layers.9.mlp.up_proj.weight"]
    assert sorted(n for n, _, _ in err.wrong_shape) == ["model.layers.1.mlp.down_proj.weight",
                                                         "model.layers.2.self_attn.q_norm.weight"]
    msg = str(err)
    for needle in ("missing", "unexpected", "wrong shapes", "k_proj", "inv_freq", "[96, 161]", "[96, 160]"):
        assert needle in msg


def test_tied_model_with_a_differing_head_is_refused(tmp_path):
    folder = _folder(tmp_path, "a")
    path = os.path.join(folder, "model.safetensors")
    t = load_file(path)
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    save_file(t, path)
    _load(folder)                                     # an equal copy is accepted
    t["lm_head.weight"] = t["lm_head.weight"] + 1
    save_file(t, path)
    with pytest.raises(WeightError, match="tied"):
        _load(folder)


def test_no_safetensors_file(tmp_path):
    folder = _folder(tmp_path, "a")
    os.remove(os.path.join(folder, "model.safetensors"))
    with pytest.raises(WeightError, match="safetensors"):
        _load(folder)


def test_several_files_are_read(tmp_path):
    folder = _folder(tmp_path, "a")
    path = os.path.join(folder, "model.safetensors")
    t = load_file(path)
    names = sorted(t)
    os.remove(path)
    save_file({n: t[n] for n in names[::2]}, os.path.join(folder, "model-00001-of-00002.safetensors"))
    save_file({n: t[n] for n in names[1::2]}, os.path.join(folder, "model-00002-of-00002.safetensors"))
    m = _load(folder)
    assert torch.equal(m.params["model.norm.weight"], t["model.norm.weight"])
