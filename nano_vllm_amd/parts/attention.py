"""Mixer parts.

"attention": grouped-query causal attention over a paged cache
(nanovllm/models/qwen3.py:14-88, nanovllm/layers/attention.py:43-75):
    qkv = x Wqkv^T (+ b)            rows of Wqkv: q heads, k heads, v heads (linear.py:111-128)
    q, k <- per-head RMS norm       when qk_norm (qwen3.py:68-70,82-84)
    q, k <- position encoding       (qwen3.py:85)
    cache <- k, v                   (attention.py:62-63)
    o = softmax(scale q K^T) V      causal, over the request's cached keys, optionally a window
    out = o Wo^T                    (qwen3.py:87)

Interface of a mixer:
    cache_need()                 -> PagedKV | FixedState | None
    forward(x [T, hidden], batch, cache) -> [T, hidden]
`cache` is the run's LayerCache (its tensors and the index of its group in batch.groups).
"""
from __future__ import annotations

from typing import Dict, Mapping

from .base import BuildContext, ParamDecl, Part, Source
from .registry import register_part
from .spec import PagedKV


class Attention(Part):
    """params: hidden_size, num_heads, num_kv_heads, head_dim, qk_norm (bool), eps, bias (bool),
    position_encoding (a name in the model's position encodings, or None), window (None or
    keys), scale (None: head_dim^-0.5), reads_shared_cache (bool: the run owns no cache, it
    projects q only and reads another run's keys and values)."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        p = params
        self.hidden = int(p["hidden_size"])
        self.heads = int(p["num_heads"])
        self.kv_heads = int(p["num_kv_heads"])
        self.head_dim = int(p["head_dim"])
        if self.heads % self.kv_heads:
            raise ValueError(f"attention: {self.heads} heads do not divide into {self.kv_heads} kv heads")
        self.qk_norm = bool(p.get("qk_norm", False))
        self.eps = float(p.get("eps", 1e-6))
        self.bias = bool(p.get("bias", False))
        self.window = p.get("window")
        scale = p.get("scale")
        self.scale = float(scale) if scale is not None else self.head_dim ** -0.5     # qwen3.py:39
        self.shared = bool(p.get("reads_shared_cache", False))
        name = p.get("position_encoding")
        self.position_encoding = build.position_encodings[name] if name else None
        self.q_name, self.k_name, self.v_name = (p.get("q_name", "q_proj"), p.get("k_name", "k_proj"),
                                                 p.get("v_name", "v_proj"))
        self.o_name = p.get("o_name", "o_proj")

    # ------------------------------------------------------------------ declaration
    def param_decls(self) -> Dict[str, ParamDecl]:
        q, kv, h = self.heads * self.head_dim, self.kv_heads * self.head_dim, self.hidden
        d: Dict[str, ParamDecl] = {}
        if self.shared:
            shards = ((self.q_name, 0, q),)
            rows = q
        else:
            shards = ((self.q_name, 0, q), (self.k_name, q, kv), (self.v_name, q + kv, kv))
            rows = q + 2 * kv
        d["qkv_proj.weight"] = ParamDecl((rows, h), sources=tuple(Source(f"{n}.weight", r, c) for n, r, c in shards))
        if self.bias:
            d["qkv_proj.bias"] = ParamDecl((rows,), sources=tuple(Source(f"{n}.bias", r, c) for n, r, c in shards))
        if self.qk_norm:
            d["q_norm.weight"] = ParamDecl((self.head_dim,), dtype="stored32", init="norm")
            if not self.shared:
                d["k_norm.weight"] = ParamDecl((self.head_dim,), dtype="stored32", init="norm")
        d[f"{self.o_name}.weight"] = ParamDecl((h, q))
        return d

    def cache_need(self):
        if self.shared:
            return None
        return PagedKV(self.kv_heads, self.head_dim, self.window)

    # ------------------------------------------------------------------ forward
    def forward(self, x, batch, cache):
        k = self.kernels
        w = self.weights
        kv_heads = 0 if self.shared else self.kv_heads
        # deferred: the products below are handed to the q/k preparation and to the block's norm only
        pe = self.position_encoding
        table = pe.rotary_table() if pe is not None else None
        qkv = k.linear(x, w["qkv_proj.weight"], w.get("qkv_proj.bias"), deferred=pe is None or table is not None)
        group = batch.groups[cache.group]
        slots = None if self.shared else group.slot_mapping
        kc, vc = (None, None) if self.shared else (cache.k, cache.v)
        qw = w.get("q_norm.weight")
        kw = w.get("k_norm.weight")
        if pe is None or table is not None:
            q = k.qk_norm_rope_store(qkv, self.heads, kv_heads, self.head_dim, qw, kw, self.eps, table,
                                     batch.positions, slots, kc, vc, max_position=batch.max_kv_len)
        else:
            # an encoding without a table: norm, the part's own encoding, then the store
            q = k.qk_norm_rope_store(qkv, self.heads, kv_heads, self.head_dim, qw, kw, self.eps, None, None,
                                     None, None, None)
            qd = self.heads * self.head_dim
            pe.apply(q, qkv[:, qd: qd + kv_heads * self.head_dim], batch.positions, self.heads, kv_heads,
                     self.head_dim)
            if not self.shared:
                k.qk_norm_rope_store(qkv, self.heads, kv_heads, self.head_dim, None, None, self.eps, None, None,
                                     slots, kc, vc)
        o = k.paged_attention(q, self.heads, self.kv_heads, self.head_dim, cache.k, cache.v, batch, cache.group,
                              self.scale, self.window)
        return k.linear(o, w[f"{self.o_name}.weight"], deferred=True)


register_part("mixer", "attention", Attention)
