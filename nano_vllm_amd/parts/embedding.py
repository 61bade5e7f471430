"""Token embedding and output head: the two ends of the model, parts like the others.

An embedding kind gives `forward(ids int32 [T]) -> [T, hidden]` and keeps its table in
`weights["weight"]`; a head kind gives `forward(x [R, hidden]) -> float32 [R, vocab]` and an
attribute `tied`: when true it declares no tensor of its own and the model hands it the
embedding's table as `weights["weight"]`.  Both are built with the model's `vocab_size` and
`hidden_size` added to their parameters.
"""
from __future__ import annotations

from typing import Mapping

from .base import BuildContext, ParamDecl, Part
from .registry import register_part


class TokenEmbedding(Part):
    """weight [vocab, hidden]; rows are gathered by token id (embed_head.py:24,38)."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        self.vocab, self.hidden = int(params["vocab_size"]), int(params["hidden_size"])

    def param_decls(self):
        return {"weight": ParamDecl((self.vocab, self.hidden))}

    def forward(self, ids):
        return self.kernels.embedding(self.weights["weight"], ids)


class OutputHead(Part):
    """logits = x W^T in float32, W [vocab, hidden] (embed_head.py:61); tied: W is the
    embedding's storage and the checkpoint holds no tensor for it (qwen3.py:202-203)."""

    def __init__(self, params: Mapping, build: BuildContext):
        super().__init__(params, build)
        self.vocab, self.hidden = int(params["vocab_size"]), int(params["hidden_size"])
        self.tied = bool(params.get("tied", False))

    def param_decls(self):
        return {} if self.tied else {"weight": ParamDecl((self.vocab, self.hidden))}

    def forward(self, x):
        return self.kernels.linear(x, self.weights["weight"], out_float32=True)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "output_head", OutputHead)
