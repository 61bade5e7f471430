"""Typed model configuration, read from the architecture's own config.json keys.

Reference: the keys that nanovllm/models/qwen3.py:128-144,169-171,201-202 and
nanovllm/engine/model_runner.py:29,110-112 read from the Hugging Face config object.
Nothing here imports transformers: config.json is parsed as plain JSON.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, asdict, fields
from typing import Any, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """config.json is missing a key, or holds a value the engine cannot honour."""


_DTYPE_NAMES = {
    "bfloat16": "bfloat16", "bf16": "bfloat16", "torch.bfloat16": "bfloat16",
    "float32": "float32", "fp32": "float32", "float": "float32", "torch.float32": "float32",
    "float16": "float16", "fp16": "float16", "half": "float16", "torch.float16": "float16",
}


def canonical_dtype(name: str) -> str:
    try:
        return _DTYPE_NAMES[str(name)]
    except KeyError:
        raise ConfigError(f"unknown dtype {name!r}; known: {sorted(set(_DTYPE_NAMES.values()))}")


def _require(d: Mapping[str, Any], key: str, typ, where: str):
    if key not in d or d[key] is None:
        raise ConfigError(f"{where}: required key {key!r} is missing")
    v = d[key]
    if typ is int and (isinstance(v, bool) or not isinstance(v, int)):
        raise ConfigError(f"{where}: key {key!r} must be an integer, got {v!r}")
    if typ is float and (isinstance(v, bool) or not isinstance(v, (int, float))):
        raise ConfigError(f"{where}: key {key!r} must be a number, got {v!r}")
    return typ(v)


@dataclass(frozen=True)
class Qwen3Config:
    """Qwen3 dense decoder.  Field names are config.json's own."""
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool = False
    attention_bias: bool = False
    hidden_act: str = "silu"
    dtype: str = "bfloat16"
    eos_token_id: Optional[Tuple[int, ...]] = None
    architecture: str = "Qwen3ForCausalLM"

    # ------------------------------------------------------------------ parsing
    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Qwen3Config":
        where = "config.json"
        hidden = _require(d, "hidden_size", int, where)
        heads = _require(d, "num_attention_heads", int, where)
        kv_heads = _require(d, "num_key_value_heads", int, where)
        # head_dim absent or null -> hidden // heads (qwen3.py:36,134)
        head_dim = d.get("head_dim")
        if head_dim is None:
            if hidden % heads:
                raise ConfigError(f"{where}: head_dim is absent and hidden_size {hidden} is "
                                  f"not a multiple of num_attention_heads {heads}")
            head_dim = hidden // heads
        # rope_theta default 1e6 (qwen3.py:135); a rope_scaling dict may carry only a
        # rope_theta of its own (qwen3.py:54-55) - the reference applies no other scaling.
        theta = d.get("rope_theta", 1000000.0)
        scaling = d.get("rope_scaling")
        if isinstance(scaling, dict):
            other = {k: v for k, v in scaling.items()
                     if k not in ("rope_theta", "rope_type", "type") and v is not None}
            kind = scaling.get("rope_type", scaling.get("type", "default"))
            if other or kind not in ("default", None):
                raise ConfigError(f"{where}: rope_scaling {scaling!r} asks for scaled rotary "
                                  "frequencies, which this architecture's engine does not apply")
            theta = scaling.get("rope_theta", theta)
        elif scaling is not None:
            raise ConfigError(f"{where}: rope_scaling must be null or an object, got {scaling!r}")
        if d.get("use_sliding_window"):
            raise ConfigError(f"{where}: use_sliding_window=true is not honoured by this "
                              "architecture (the reference reads no window key); refusing "
                              "rather than attending to all keys silently")
        act = d.get("hidden_act", "silu")
        if act != "silu":                                          # qwen3.py:110
            raise ConfigError(f"{where}: hidden_act must be 'silu', got {act!r}")
        dtype = canonical_dtype(d.get("dtype") or d.get("torch_dtype") or "bfloat16")
        eos = d.get("eos_token_id")
        if isinstance(eos, int):
            eos = (eos,)
        elif isinstance(eos, (list, tuple)):
            eos = tuple(int(x) for x in eos)
        else:
            eos = None
        cfg = cls(
            vocab_size=_require(d, "vocab_size", int, where),
            hidden_size=hidden,
            num_hidden_layers=_require(d, "num_hidden_layers", int, where),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=int(head_dim),
            intermediate_size=_require(d, "intermediate_size", int, where),
            rms_norm_eps=_require(d, "rms_norm_eps", float, where),
            rope_theta=float(theta),
            max_position_embeddings=_require(d, "max_position_embeddings", int, where),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            # The reference's getattr default is True (qwen3.py:133); every Qwen3 file
            # states false, so an absent key means no bias here.
            attention_bias=bool(d.get("attention_bias", False)),
            hidden_act=act,
            dtype=dtype,
            eos_token_id=eos,
            architecture=(d.get("architectures") or ["Qwen3ForCausalLM"])[0],
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for f in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                  "num_key_value_heads", "head_dim", "intermediate_size",
                  "max_position_embeddings"):
            if getattr(self, f) <= 0:
                raise ConfigError(f"config.json: {f} must be positive, got {getattr(self, f)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: num_attention_heads {self.num_attention_heads} is not a multiple "
                f"of num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim {self.head_dim} must be even for rotary pairs")
        if not (self.rms_norm_eps > 0):
            raise ConfigError(f"config.json: rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if not (self.rope_theta > 0):
            raise ConfigError(f"config.json: rope_theta must be positive, got {self.rope_theta}")

    def to_dict(self) -> dict:
        """The config.json that describes this configuration."""
        d = asdict(self)
        arch = d.pop("architecture")
        dtype = d.pop("dtype")
        eos = d.pop("eos_token_id")
        out = {"architectures": [arch], "model_type": "qwen3"}
        out.update(d)
        out["torch_dtype"] = dtype
        out["rope_scaling"] = None
        out["use_sliding_window"] = False
        if eos is not None:
            out["eos_token_id"] = eos[0] if len(eos) == 1 else list(eos)
        return out

    def replace(self, **kw) -> "Qwen3Config":
        d = {f.name: getattr(self, f.name) for f in fields(self)}
        d.update(kw)
        return Qwen3Config(**d)


def read_config_json(folder: str) -> dict:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{folder!r} holds no config.json")
    with open(path) as f:
        return json.load(f)
