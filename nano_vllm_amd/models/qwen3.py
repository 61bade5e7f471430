"""Qwen3 dense decoder as data: config.json -> typed configuration -> ModelSpec.

Reference: nanovllm/models/qwen3.py.  Every layer is the pre-norm residual block of
qwen3.py:121-159 with grouped-query attention (per-head q/k norm when there is no bias,
qwen3.py:68-70; rotary pairs (i, i+D/2), one table shared by all layers, rotary_embedding.py:51-59)
and the SwiGLU feed-forward of qwen3.py:91-117.  Tensor names are the checkpoint's
(qwen3.py:42,49,69-70,100,105,143-144,169-171,200-201 and the packing of qwen3.py:187-193).
"""
from __future__ import annotations

from ..config.model_config import Qwen3Config
from ..config.registry import register_architecture
from ..parts.spec import LayerRun, LayerSpec, ModelSpec, PartSpec


def build_spec(cfg: Qwen3Config) -> ModelSpec:
    norm = {"dim": cfg.hidden_size, "eps": cfg.rms_norm_eps}
    mixer = PartSpec("attention", {
        "hidden_size": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
        "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
        "qk_norm": not cfg.attention_bias,         # qwen3.py:68
        "eps": cfg.rms_norm_eps, "bias": cfg.attention_bias,
        "position_encoding": "rotary", "window": None, "scale": None,
    })
    ffn = PartSpec("swiglu", {"hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size})
    layers = tuple(
        LayerSpec(
            block=PartSpec("pre_norm_residual"),
            parts={"mixer_norm": PartSpec("rms_norm", norm), "mixer": mixer,
                   "feed_forward_norm": PartSpec("rms_norm", norm), "feed_forward": ffn},
            name=f"model.layers.{i}",
            names={"mixer_norm": "input_layernorm", "mixer": "self_attn",
                   "feed_forward_norm": "post_attention_layernorm", "feed_forward": "mlp"},
        ) for i in range(cfg.num_hidden_layers))
    return ModelSpec(
        architecture=cfg.architecture,
        hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size,
        max_position=cfg.max_position_embeddings, dtype=cfg.dtype,
        embedding=PartSpec("token_embedding", {"name": "model.embed_tokens"}),
        layers=layers,
        order=tuple(LayerRun(i) for i in range(cfg.num_hidden_layers)),
        final_norm=PartSpec("rms_norm", {**norm, "name": "model.norm"}),
        head=PartSpec("output_head", {"name": "lm_head", "tied": cfg.tie_word_embeddings}),
        position_encodings={"rotary": PartSpec("rotary_neox", {
            "head_dim": cfg.head_dim, "theta": cfg.rope_theta, "max_position": cfg.max_position_embeddings})},
        eos_token_ids=cfg.eos_token_id or (),
    )


register_architecture("Qwen3ForCausalLM", Qwen3Config.from_dict, build_spec, replace=True)
