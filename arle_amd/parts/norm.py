"""Norms over the model width.  RMSNorm: x / sqrt(mean(x^2) + eps) * w with the plain weight w (not 1 + w);
LayerNorm without bias.

crates/cuda-kernels/csrc/misc/norm.cu:8,59,221-359; the residual add fused in as at :462-.
The weight keeps the type the checkpoint stores it in (bfloat16 or float32).
"""
from __future__ import annotations

from ..kernels import ops
from .base import Part, WeightDecl, register


@register("norm", "rmsnorm")
class RMSNorm(Part):
    """params: width, eps."""

    graph_safe = True  # launches depend on shapes only, never on the values of a step

    @classmethod
    def declare_weights(cls, params):
        return {"weight": WeightDecl((params["width"],), init="ones")}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.weight = tensors["weight"]
        self.eps = float(params["eps"])
        self.width = int(params["width"])

    def forward(self, x, rows=None):
        return ops.rmsnorm(x, self.weight, self.eps, self.rt.act_dtype, rows=rows)

    def add_norm(self, residual, delta, rows=None):
        """residual (float32) += delta, then the norm of it; delta None: just the norm."""
        if delta is None:
            return ops.rmsnorm(residual, self.weight, self.eps, self.rt.act_dtype, rows=rows)
        return ops.add_rmsnorm(residual, delta, self.weight, self.eps, self.rt.act_dtype, rows=rows)


@register("norm", "layernorm")
class LayerNorm(Part):
    """(x - mean) / sqrt(var + eps) * w, var the mean of the squared deviations, no bias.  params: width, eps.

    `add_norm` takes what the block before has left to add as one tensor, one float32 stack of partial sums, or a
    `Pending` list of up to two of them, each with the bias of the projection that made it; with `also`, a second
    norm of the same sum (another weight, the same width and eps) comes out of the same pass: the two norms of a
    block whose mixer and feed-forward read the same residual."""

    graph_safe = True  # launches depend on shapes only, never on the values of a step

    @classmethod
    def declare_weights(cls, params):
        return {"weight": WeightDecl((params["width"],), init="ones")}

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.weight = tensors["weight"]
        self.eps = float(params["eps"])
        self.width = int(params["width"])

    def forward(self, x, rows=None):
        return self.add_norm(x, None, rows=rows)

    def add_norm(self, residual, delta, rows=None, also=None):
        terms = delta if isinstance(delta, list) else ([] if delta is None else [(delta, None)])
        if also is not None and (also.eps != self.eps or also.width != self.width):
            raise ValueError("two norms share a pass only with one width and one eps")
        return ops.add_layernorm(residual, terms, self.weight, self.eps, self.rt.act_dtype,
                                 weight_b=also.weight if also is not None else None, rows=rows)
