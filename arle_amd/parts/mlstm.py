"""The mLSTM mixer: a matrix memory per head with exponential input and forget gates in log space, kept stable
by a running maximum, as in xLSTM.

Per token, with h the mixer's input, H heads, key size D, value size Dv:

    q = W_q h * D^(-1/2),  k = W_k h,  v = W_v h
    i = cap tanh((W_i h + b_i) / cap),   f = logsigmoid(cap tanh((W_f h + b_f) / cap))         (per head)
    m' = max(f + m, i);  S' = exp(f + m - m') S + exp(i - m') k v^T;  n' likewise with k alone
    o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
    out = W_o ((o / rms(o) per head) * w_norm * sigmoid(W_g h))

S, n and m start at zero and live in 32-bit state slots `[H, D, Dv]`, `[H, D]`, `[H]` of the request; the gates'
projections, the gates, the recurrence and the head norm are 32-bit in every mode.  q, k, v and the output gate
come from one fused product that hands over its 32-bit sums; the two gate projections are a product of their own.
"""
from __future__ import annotations

import torch

from ..cache.manager import StateNeed
from ..kernels import ops
from .base import Part, WeightDecl, register
from .linear import Linear


@register("mixer", "mlstm")
class MLSTMMixer(Part):
    """params: hidden_size, heads, key_dim, value_dim, gate_cap, eps."""

    graph_safe = True  # rows, slots and lengths are read on the GPU; launches depend on shapes only

    @classmethod
    def declare_weights(cls, params):
        w, h, d, dv = params["hidden_size"], params["heads"], params["key_dim"], params["value_dim"]
        return {"q": WeightDecl((h * d, w)), "k": WeightDecl((h * d, w)), "v": WeightDecl((h * dv, w)),
                "g": WeightDecl((h * dv, w)), "o": WeightDecl((w, h * dv)), "norm": WeightDecl((h * dv,), init="ones"),
                "i": WeightDecl((h, w)), "i_bias": WeightDecl((h,), init="normal"),
                "f": WeightDecl((h, w)), "f_bias": WeightDecl((h,), init="normal")}

    @classmethod
    def declare_cache(cls, params):
        h, d, dv = int(params["heads"]), int(params["key_dim"]), int(params["value_dim"])
        return {"S": StateNeed((h, d, dv), torch.float32), "n": StateNeed((h, d), torch.float32),
                "m": StateNeed((h,), torch.float32)}

    def cache_need(self):
        return self.declare_cache(self.params)

    def __init__(self, params, tensors, rt, children=None):
        super().__init__(params, tensors, rt, children)
        self.H, self.D, self.Dv = int(params["heads"]), int(params["key_dim"]), int(params["value_dim"])
        if not 0 < self.D <= ops.MLSTM_MAX_KEY_DIM:
            raise ValueError(f"key_dim {self.D} is not supported: the mLSTM kernels take 1..{ops.MLSTM_MAX_KEY_DIM}")
        self.cap = float(params["gate_cap"])
        self.eps = float(params["eps"])
        fused = [tensors[n] for n in ("q", "k", "v", "g")]
        if len({t.dtype for t in fused}) != 1:
            raise ValueError("q, k, v and gate projections must be stored in one type")
        self.qkvg = Linear(torch.cat(fused, dim=0).contiguous(), rt.weight_tiles)
        # The gates enter the recurrence: their projection hands over 32-bit sums whatever the mode.  In bfloat16 it
        # is a product of bfloat16 operands like every projection (rows padded with zeros to whole tiles of 16 outputs),
        # in float32 the fixed-order 32-bit product.
        gates = torch.cat([tensors["i"], tensors["f"]], dim=0)
        if gates.dtype == torch.bfloat16 and not rt.is_f32:
            pad = -gates.shape[0] % 16
            gates = torch.cat([gates, gates.new_zeros((pad, gates.shape[1]))], dim=0) if pad else gates
            self.gates = Linear(gates.contiguous(), rt.weight_tiles)
        else:
            self.gates = Linear(gates.float().contiguous())
        self.i_bias, self.f_bias = tensors["i_bias"].float().contiguous(), tensors["f_bias"].float().contiguous()
        self.norm = tensors["norm"]
        self.o = Linear(tensors["o"], rt.weight_tiles)

    def products(self):
        if self.qkvg.weight.dtype != torch.bfloat16:
            return []
        return [("qkvg", self.qkvg.out_features, self.qkvg.in_features, False, None),
                ("o", self.o.out_features, self.o.in_features, False, "norm")]

    def forward(self, x, batch, cache):
        """x [T, W] -> [T, W], or a float32 stack [S, T, W] to be added in order (see Linear)."""
        qk, vw = self.H * self.D, self.H * self.Dv
        # 32-bit sums out of the product: q and k meet in dot products whose terms cancel (a request's first rows hang
        # on a single one), and what rounding them to bfloat16 costs there is ten times a usual row's error
        p = self.qkvg(x, out_dtype=torch.float32)
        q, k, v, g = p[:, :qk], p[:, qk:2 * qk], p[:, 2 * qk:2 * qk + vw], p[:, 2 * qk + vw:]
        gates = self.gates(x, out_dtype=torch.float32)[:, :2 * self.H]
        num, nq, coefs = ops.mlstm_scan(q, k, v, gates, self.i_bias, self.f_bias, self.cap, cache["S"].state,
                                        cache["n"].state, cache["m"].state, batch.seg_row0, batch.seg_slot,
                                        heads=self.H, key_dim=self.D, value_dim=self.Dv)
        y = ops.mlstm_output(num, nq, coefs, g, self.norm, self.eps, self.rt.act_dtype, heads=self.H, value_dim=self.Dv)
        return self.o(y, out_dtype=torch.float32, partials_ok=True)   # it goes into the 32-bit residual unrounded
