"""Named config.json contents for runs with random weights (there is no checkpoint to read
them from): two tiny test shapes and the Qwen3 dense sizes that the benchmarks use.  These are
inputs, as a model folder's config.json is; nothing in the model code reads them.

    python -m nano_vllm_amd.cli random-model --shape qwen3-8b --config-only --out DIR
    python -m nano_vllm_amd.cli throughput --model DIR --random-weights 0
"""
from __future__ import annotations

from typing import Dict


def _qwen3(layers, hidden, heads, kv_heads, head_dim, inner, vocab, theta=1e6, eps=1e-6, tied=False,
           max_position=40960, dtype="bfloat16") -> dict:
    return {"architectures": ["Qwen3ForCausalLM"], "hidden_size": hidden, "num_hidden_layers": layers,
            "num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": head_dim,
            "intermediate_size": inner, "vocab_size": vocab, "rms_norm_eps": eps, "rope_theta": theta,
            "max_position_embeddings": max_position, "tie_word_embeddings": tied, "attention_bias": False,
            "hidden_act": "silu", "torch_dtype": dtype}


SHAPES: Dict[str, dict] = {
    "tiny-a": _qwen3(2, 64, 4, 2, 16, 128, 256, theta=1e4, tied=True, max_position=128, dtype="float32"),
    "tiny-b": _qwen3(3, 96, 8, 2, 32, 160, 384, eps=1e-5, max_position=256, dtype="float32"),
    "qwen3-0.6b": _qwen3(28, 1024, 16, 8, 128, 3072, 151936, tied=True),     # the model of the reference's README benchmark
    "qwen3-1.7b": _qwen3(28, 2048, 16, 8, 128, 6144, 151936, tied=True),
    "qwen3-4b": _qwen3(36, 2560, 32, 8, 128, 9728, 151936, tied=True),
    "qwen3-8b": _qwen3(36, 4096, 32, 8, 128, 12288, 151936),
    "qwen3-14b": _qwen3(40, 5120, 40, 8, 128, 17408, 151936),
    "qwen3-32b": _qwen3(64, 5120, 64, 8, 128, 25600, 151936),
}


def shape(name: str) -> dict:
    if name not in SHAPES:
        raise KeyError(f"unknown shape {name!r}; known: {sorted(SHAPES)}")
    return dict(SHAPES[name])
