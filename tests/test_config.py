"""Configuration: config.json keys, defaults, refusals, registry, engine options."""
import json
import os

import pytest

from nano_vllm_amd.config import (ConfigError, EngineConfig, Qwen3Config, architecture_of, get_architecture,
                                  known_architectures, register_architecture)

# keys as a Qwen3 checkpoint's config.json carries them
QWEN3_JSON = {
    "architectures": ["Qwen3ForCausalLM"], "attention_bias": False, "attention_dropout": 0.0,
    "bos_token_id": 151643, "eos_token_id": 151645, "head_dim": 128, "hidden_act": "silu",
    "hidden_size": 1024, "initializer_range": 0.02, "intermediate_size": 3072,
    "max_position_embeddings": 40960, "max_window_layers": 28, "model_type": "qwen3",
    "num_attention_heads": 16, "num_hidden_layers": 28, "num_key_value_heads": 8,
    "rms_norm_eps": 1e-06, "rope_scaling": None, "rope_theta": 1000000, "sliding_window": None,
    "tie_word_embeddings": True, "torch_dtype": "bfloat16", "use_cache": True,
    "use_sliding_window": False, "vocab_size": 151936,
}


def test_parses_a_checkpoint_config():
    c = Qwen3Config.from_dict(QWEN3_JSON)
    assert (c.hidden_size, c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (1024, 16, 8, 128)
    assert c.head_dim * c.num_attention_heads != c.hidden_size          # q width differs from hidden
    assert c.tie_word_embeddings and not c.attention_bias
    assert c.dtype == "bfloat16" and c.rope_theta == 1e6 and c.eos_token_id == (151645,)


def test_defaults():
    d = {k: v for k, v in QWEN3_JSON.items() if k not in ("head_dim", "rope_theta", "tie_word_embeddings",
                                                          "torch_dtype", "attention_bias", "eos_token_id")}
    c = Qwen3Config.from_dict(d)
    assert c.head_dim == 1024 // 16                # qwen3.py:36
    assert c.rope_theta == 1e6                     # qwen3.py:135
    assert c.tie_word_embeddings is False and c.attention_bias is False and c.dtype == "bfloat16"
    assert c.eos_token_id is None


def test_dtype_key_and_eos_list():
    d = dict(QWEN3_JSON, dtype="float32", eos_token_id=[1, 2])
    d.pop("torch_dtype")
    c = Qwen3Config.from_dict(d)
    assert c.dtype == "float32" and c.eos_token_id == (1, 2)


@pytest.mark.parametrize("key", ["hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
                                 "intermediate_size", "vocab_size", "rms_norm_eps", "max_position_embeddings"])
def test_missing_required_key_is_named(key):
    d = dict(QWEN3_JSON)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(d)


def test_refusals():
    with pytest.raises(ConfigError, match="hidden_act"):
        Qwen3Config.from_dict(dict(QWEN3_JSON, hidden_act="gelu"))
    with pytest.raises(ConfigError, match="sliding"):
        Qwen3Config.from_dict(dict(QWEN3_JSON, use_sliding_window=True))
    with pytest.raises(ConfigError, match="rope_scaling"):
        Qwen3Config.from_dict(dict(QWEN3_JSON, rope_scaling={"rope_type": "yarn", "factor": 4.0}))
    with pytest.raises(ConfigError, match="multiple"):
        Qwen3Config.from_dict(dict(QWEN3_JSON, num_attention_heads=16, num_key_value_heads=5))
    with pytest.raises(ConfigError, match="dtype"):
        Qwen3Config.from_dict(dict(QWEN3_JSON, torch_dtype="int8"))
    with pytest.raises(ConfigError, match="integer"):
        Qwen3Config.from_dict(dict(QWEN3_JSON, hidden_size="1024"))


def test_rope_scaling_may_carry_a_theta_of_its_own():
    c = Qwen3Config.from_dict(dict(QWEN3_JSON, rope_scaling={"rope_theta": 5000.0}))      # qwen3.py:54-55
    assert c.rope_theta == 5000.0


def test_round_trip_through_config_json():
    c = Qwen3Config.from_dict(QWEN3_JSON)
    assert Qwen3Config.from_dict(json.loads(json.dumps(c.to_dict()))) == c


def test_registry():
    assert "Qwen3ForCausalLM" in known_architectures()
    arch = architecture_of(QWEN3_JSON)
    spec = arch.build_spec(arch.parse_config(QWEN3_JSON))
    assert len(spec.layers) == 28 and len(spec.order) == 28 and spec.head["tied"]
    mixer = spec.layers[0].parts["mixer"]
    assert mixer.kind == "attention" and mixer["qk_norm"] and mixer["window"] is None
    with pytest.raises(ConfigError, match="LlamaForCausalLM.*Qwen3ForCausalLM"):
        get_architecture("LlamaForCausalLM")
    with pytest.raises(ConfigError, match="architectures"):
        architecture_of({})
    with pytest.raises(ValueError, match="already"):
        register_architecture("Qwen3ForCausalLM", None, None)


def test_no_size_is_fixed_in_the_spec():
    d = dict(QWEN3_JSON, hidden_size=120, num_attention_heads=6, num_key_value_heads=3, head_dim=48,
             intermediate_size=200, vocab_size=1001, num_hidden_layers=5, rms_norm_eps=3e-5, rope_theta=777.0,
             tie_word_embeddings=False, max_position_embeddings=99)
    arch = architecture_of(d)
    spec = arch.build_spec(arch.parse_config(d))
    m = spec.layers[4].parts["mixer"]
    assert (m["hidden_size"], m["num_heads"], m["num_kv_heads"], m["head_dim"], m["eps"]) == (120, 6, 3, 48, 3e-5)
    assert spec.layers[4].parts["feed_forward"]["intermediate_size"] == 200
    assert spec.position_encodings["rotary"]["theta"] == 777.0
    assert spec.position_encodings["rotary"]["max_position"] == 99
    assert spec.final_norm["eps"] == 3e-5 and spec.vocab_size == 1001 and not spec.head["tied"]


def test_engine_config(tmp_path):
    c = EngineConfig(str(tmp_path))
    assert (c.max_num_batched_tokens, c.max_num_seqs, c.max_model_len, c.kvcache_block_size) == (16384, 512, 4096, 256)
    assert c.gpu_memory_utilization == 0.9 and c.enforce_eager is False and c.eos == -1
    assert EngineConfig(str(tmp_path), kvcache_block_size=4).kvcache_block_size == 4       # the reference needs % 256
    with pytest.raises(ConfigError, match="exist"):
        EngineConfig(os.path.join(str(tmp_path), "nope"))
    with pytest.raises(ConfigError, match="one GPU"):
        EngineConfig(str(tmp_path), tensor_parallel_size=2)
    with pytest.raises(ConfigError):
        EngineConfig(str(tmp_path), kvcache_block_size=0)
    with pytest.raises(ConfigError, match="dtype"):
        EngineConfig(str(tmp_path), dtype="float16")
    assert EngineConfig(str(tmp_path), dtype="bf16").dtype == "bfloat16"
