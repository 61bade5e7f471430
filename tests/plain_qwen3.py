"""Plain, slow implementation of the Qwen3 dense decoder: whole sequences, no cache.

Written from the formulas in the reference's text (each function cites file:line
as nanovllm/...).  It shares no code with the engine: it reads config.json
and model.safetensors itself, keeps q/k/v and gate/up as separate matrices, builds
a dense causal mask and recomputes everything for every call.

``rounding`` selects where results are rounded:
  * ``None``     - everything in the tensors' own dtype (float32 or float64);
  * ``bfloat16`` - float32 arithmetic with a rounding to bfloat16 at every place
                   where the reference, run with a bfloat16 model, materialises a
                   bfloat16 tensor.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass

import torch
from safetensors import safe_open


# --------------------------------------------------------------------------- config

@dataclass
class PlainConfig:
    vocab_size: int
    hidden_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    rms_norm_eps: float
    rope_theta: float
    max_position: int
    tie_word_embeddings: bool
    attention_bias: bool

    @staticmethod
    def from_dict(d: dict) -> "PlainConfig":
        heads = d["num_attention_heads"]
        # head_dim: qwen3.py:36,134 (absent -> hidden_size // heads)
        head_dim = d.get("head_dim") or d["hidden_size"] // heads
        theta = d.get("rope_theta", 1000000)                      # qwen3.py:135
        scaling = d.get("rope_scaling")
        if isinstance(scaling, dict):                             # qwen3.py:54-55
            theta = scaling.get("rope_theta", theta)
        assert d.get("hidden_act", "silu") == "silu"              # qwen3.py:110
        return PlainConfig(
            vocab_size=d["vocab_size"], hidden_size=d["hidden_size"],
            num_layers=d["num_hidden_layers"], num_heads=heads,
            num_kv_heads=d["num_key_value_heads"], head_dim=head_dim,
            intermediate_size=d["intermediate_size"], rms_norm_eps=d["rms_norm_eps"],
            rope_theta=float(theta), max_position=d["max_position_embeddings"],
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            attention_bias=bool(d.get("attention_bias", False)),
        )


def read_folder(path: str, dtype=torch.float32):
    """config.json + every tensor of model.safetensors, cast to ``dtype``."""
    with open(os.path.join(path, "config.json")) as f:
        cfg = PlainConfig.from_dict(json.load(f))
    weights = {}
    with safe_open(os.path.join(path, "model.safetensors"), "pt", "cpu") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).to(dtype)
    return cfg, weights


# --------------------------------------------------------------------------- rounding

def _rounder(rounding):
    if rounding is None:
        return lambda x: x
    assert rounding == "bfloat16"
    return lambda x: x.to(torch.bfloat16).to(x.dtype)


# --------------------------------------------------------------------------- parts

def rms_norm(x, weight, eps, rounding=None):
    """layernorm.py:16-26.  var = mean(x^2); x * rsqrt(var + eps); cast; * weight."""
    rd = _rounder(rounding)
    var = x.pow(2).mean(dim=-1, keepdim=True)
    y = x * torch.rsqrt(var + eps)
    return rd(rd(y) * weight)            # the cast precedes the weight (layernorm.py:25)


def add_rms_norm(x, residual, weight, eps, rounding=None):
    """layernorm.py:28-40.  The sum is the new residual; the variance is taken of
    the unrounded sum (layernorm.py:35-37)."""
    rd = _rounder(rounding)
    s = x + residual
    new_residual = rd(s)
    var = s.pow(2).mean(dim=-1, keepdim=True)
    y = s * torch.rsqrt(var + eps)
    return rd(rd(y) * weight), new_residual


def rope_angles(head_dim, positions, base):
    """rotary_embedding.py:29-31.  inv_freq_i = 1 / base^(2i/D); angle = p * inv_freq,
    all in float32 as in the reference's table, whatever the model dtype."""
    inv_freq = 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.float) / head_dim))
    t = positions.to(torch.float)
    return torch.einsum("i,j -> ij", t, inv_freq)          # [T, D/2]


def apply_rope(x, angles, rounding=None):
    """rotary_embedding.py:6-14.  Pairs are (i, i + D/2): first half with second half.
    x [T, heads, D]; angles [T, D/2]."""
    rd = _rounder(rounding)
    cos = angles.cos().to(x.dtype).unsqueeze(1)
    sin = angles.sin().to(x.dtype).unsqueeze(1)
    x1, x2 = torch.chunk(x, 2, dim=-1)
    y1 = x1 * cos - x2 * sin
    y2 = x2 * cos + x1 * sin
    return rd(torch.cat((y1, y2), dim=-1))


def causal_attention(q, k, v, scale, window=None, rounding=None):
    """attention.py:64-75 with causal=True; q head h reads kv head h // G (qwen3.py:62-67).
    q [T, Hq, D], k and v [T, Hkv, D].  A key j is seen from position i iff j <= i
    (and i - j < window, where a window is given)."""
    rd = _rounder(rounding)
    T, Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    out = torch.empty_like(q)
    idx = torch.arange(T)
    visible = idx[None, :] <= idx[:, None]
    if window is not None:
        visible &= (idx[:, None] - idx[None, :]) < window
    for h in range(Hq):
        kh, vh = k[:, h // G], v[:, h // G]
        s = (q[:, h] @ kh.T) * scale
        s = s.masked_fill(~visible, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, h] = p @ vh
    return rd(out)


def silu_mul(gate, up, rounding=None):
    """activation.py:8-11: silu(gate) * up, silu(g) = g * sigmoid(g)."""
    rd = _rounder(rounding)
    return rd(gate * torch.sigmoid(gate) * up)


def feed_forward(x, w_gate, w_up, w_down, rounding=None):
    """qwen3.py:113-117."""
    rd = _rounder(rounding)
    g = rd(x @ w_gate.T)
    u = rd(x @ w_up.T)
    return rd(silu_mul(g, u, rounding) @ w_down.T)


def self_attention(x, positions, w, prefix, cfg: PlainConfig, window=None, rounding=None, kv=None, keep=None):
    """qwen3.py:72-88: projections, per-head q/k norm (only without bias), rotation,
    attention, output projection.  For the tests of layer orders (not a reference feature):
    kv = (k, v) of another layer replaces this layer's own keys and values; keep, a list,
    receives this layer's (k, v)."""
    rd = _rounder(rounding)
    T = x.shape[0]
    D = cfg.head_dim

    def proj(name):
        y = x @ w[f"{prefix}.{name}.weight"].T
        if cfg.attention_bias:                                     # qwen3.py:47
            y = y + w[f"{prefix}.{name}.bias"]
        return rd(y)

    q = proj("q_proj").view(T, cfg.num_heads, D)
    if not cfg.attention_bias:                                     # qwen3.py:68-70,82-84
        q = rms_norm(q, w[f"{prefix}.q_norm.weight"], cfg.rms_norm_eps, rounding)
    angles = rope_angles(D, positions, cfg.rope_theta)
    q = apply_rope(q, angles, rounding)
    if kv is None:
        k = proj("k_proj").view(T, cfg.num_kv_heads, D)
        v = proj("v_proj").view(T, cfg.num_kv_heads, D)
        if not cfg.attention_bias:
            k = rms_norm(k, w[f"{prefix}.k_norm.weight"], cfg.rms_norm_eps, rounding)
        k = apply_rope(k, angles, rounding)
    else:
        k, v = kv
    if keep is not None:
        keep.append((k, v))
    o = causal_attention(q, k, v, D ** -0.5, window, rounding)     # qwen3.py:39
    return rd(o.reshape(T, cfg.num_heads * D) @ w[f"{prefix}.o_proj.weight"].T)


def hidden_states(w, cfg: PlainConfig, token_ids, rounding=None, first_position=0, order=None, windows=None):
    """qwen3.py:173-183 with the layer of qwen3.py:146-159.  Returns the normalised
    last hidden state of every position, [T, H].  For the tests of layer orders and windows
    (not reference features): order = [(layer, index of the earlier entry whose keys and
    values it reads, or None)], windows = {layer: keys}."""
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    positions = torch.arange(first_position, first_position + len(ids))
    h = w["model.embed_tokens.weight"][ids]                        # embed_head.py:38
    residual = None
    order = order if order is not None else [(i, None) for i in range(cfg.num_layers)]
    windows = windows or {}
    kept = []
    for i, source in order:
        p = f"model.layers.{i}"
        if residual is None:                                       # qwen3.py:152-153
            h, residual = rms_norm(h, w[f"{p}.input_layernorm.weight"], cfg.rms_norm_eps, rounding), h
        else:                                                      # qwen3.py:154-155
            h, residual = add_rms_norm(h, residual, w[f"{p}.input_layernorm.weight"],
                                       cfg.rms_norm_eps, rounding)
        h = self_attention(h, positions, w, f"{p}.self_attn", cfg, windows.get(i), rounding,
                           kv=None if source is None else kept[source], keep=kept)
        h, residual = add_rms_norm(h, residual, w[f"{p}.post_attention_layernorm.weight"],
                                   cfg.rms_norm_eps, rounding)    # qwen3.py:157
        h = feed_forward(h, w[f"{p}.mlp.gate_proj.weight"], w[f"{p}.mlp.up_proj.weight"],
                         w[f"{p}.mlp.down_proj.weight"], rounding)
    h, _ = add_rms_norm(h, residual, w["model.norm.weight"], cfg.rms_norm_eps, rounding)  # qwen3.py:182
    return h


def logits(w, cfg: PlainConfig, token_ids, rounding=None, first_position=0, order=None, windows=None):
    """Logits of every position [T, V] (embed_head.py:61; tied head: qwen3.py:202-203).
    The product with the head is left unrounded: logits are wanted in float32."""
    h = hidden_states(w, cfg, token_ids, rounding, first_position, order, windows)
    head = w["model.embed_tokens.weight"] if cfg.tie_word_embeddings else w["lm_head.weight"]
    return h @ head.T


def greedy_generate(w, cfg, prompt, num_tokens, rounding=None):
    """Token by token: the argmax at the last position of the whole, growing sequence."""
    ids = list(prompt)
    for _ in range(num_tokens):
        ids.append(int(torch.argmax(logits(w, cfg, ids, rounding)[-1])))
    return ids[len(prompt):]


# --------------------------------------------------------------------------- sampling

_M64 = (1 << 64) - 1


def _mix64(z: int) -> int:
    """The splitmix64 finaliser on Python integers."""
    z = (z + 0x9E3779B97F4A7C15) & _M64
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def exponential_noise(seed: int, request: int, position: int, vocab: int) -> torch.Tensor:
    """One Exp(1) variate per vocabulary entry, a pure function of (seed, request,
    position, entry): key = mix(mix(mix(seed) ^ request) ^ position); bits =
    mix(key ^ entry); u = (top 24 bits + 0.5) / 2^24; e = -log(u)."""
    key = _mix64(_mix64(_mix64(seed & _M64) ^ (request & _M64)) ^ (position & _M64))
    out = torch.empty(vocab, dtype=torch.float64)
    for i in range(vocab):
        bits = _mix64(key ^ i)
        u = ((bits >> 40) + 0.5) / float(1 << 24)
        out[i] = -math.log(u)
    return out


def sample(logits_row, temperature, seed=0, request=0, position=0):
    """sampler.py:8-12: argmax(softmax(l / T) / E), E ~ Exp(1); which equals
    argmax(l / T - log E).  Temperature 0 is the argmax of the logits (lowest index
    on ties)."""
    l = logits_row.to(torch.float64)
    if temperature == 0:
        return int(torch.argmax(l))
    e = exponential_noise(seed, request, position, l.numel())
    return int(torch.argmax(l / temperature - torch.log(e)))
