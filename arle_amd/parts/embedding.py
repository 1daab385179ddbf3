"""Token embedding (row gather into the 32-bit residual stream) and the output head.

infer/src/model/common.rs:64-80 (gather), :160-165 and infer/src/model/qwen3/weights.rs:305-316
(head; the embedding table itself when the two are tied -- no copy is made).
"""
from __future__ import annotations

import torch

from ..kernels import ops
from .base import Part, WeightDecl, register
from .linear import Linear


@register("embedding", "token_table")
class TokenEmbedding(Part):
    """params: vocab_size, hidden_size, scale (a factor on every row, in 32 bits; default 1)."""

    graph_safe = True  # launches depend on shapes only, never on the values of a step

    @classmethod
    def declare_weights(cls, params):
        return {"table": WeightDecl((params["vocab_size"], params["hidden_size"]))}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.table = tensors["table"]
        self.scale = float(params.get("scale", 1.0))

    def forward(self, token_ids):
        return ops.embed_gather(self.table, token_ids, scale=self.scale)


@register("head", "linear")
class LinearHead(Part):
    """params: vocab_size, hidden_size, softcap (0 or absent: none; else logits <- cap tanh(logits / cap)).
    Logits are float32."""

    graph_safe = True  # launches depend on shapes only, never on the values of a step

    @classmethod
    def declare_weights(cls, params):
        return {"weight": WeightDecl((params["vocab_size"], params["hidden_size"]))}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.proj = Linear(tensors["weight"], rt.weight_tiles)
        self.softcap = float(params.get("softcap") or 0.0)

    def products(self):
        if self.proj.weight.dtype != torch.bfloat16:
            return []
        return [("head", self.proj.out_features, self.proj.in_features, False, None)]

    def forward(self, x):
        logits = self.proj(x, out_dtype=torch.float32)
        if self.softcap > 0.0 and logits.numel():
            logits = ops.tanh_cap_(logits.contiguous(), self.softcap)
        return logits
