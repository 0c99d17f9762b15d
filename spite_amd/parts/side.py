"""What a layer adds to the stream from the step's tokens, beside its mixer and feed-forward.

``gated_token_table``: a second, narrow embedding.  Every token has a row of ``dim`` elements for
this layer in a table [V, layers * dim]; the stream gates it and a projection widens it again:

    g = gelu_tanh(W_gate x) * row[token],   y = W_proj g,   x += mult * rmsnorm(y) * w_norm

x is the stream itself (after the layer's feed-forward), not a normed copy.
"""
from __future__ import annotations

import torch

from .base import SideInput, ParamSpec, NormedIncrement, register, two_increments
from .linear import linear, Weight
from ..csrc import hipops


@register("side", "gated_token_table")
class GatedTokenTable(SideInput):
    graph_safe = True

    def __init__(self, env, vocab_size, width, dim, n_layers, layer, eps, mult=1.0):
        self.env = env
        self.V, self.d, self.dim, self.L, self.layer = int(vocab_size), int(width), int(dim), int(n_layers), int(layer)
        self.eps, self.mult = float(eps), float(mult)
        self.table = self.w_gate = self.w_proj = self.w_norm = None

    def params(self):
        return {"embed": ParamSpec((self.V, self.L * self.dim)), "gate": ParamSpec((self.dim, self.d)),
                "proj": ParamSpec((self.d, self.dim)), "norm": ParamSpec((self.d,), kind="vector", init="ones")}

    def load(self, t):
        # this layer's columns of the table, kept as a table of their own
        self.table = t["embed"][:, self.layer * self.dim:(self.layer + 1) * self.dim].contiguous()
        self.w_gate, self.w_proj = Weight(t["gate"]), Weight(t["proj"])
        self.w_norm = t["norm"].contiguous()

    def slow_paths(self, page_size):
        return self.w_gate.slow_reason("token side gate") + self.w_proj.slow_reason("token side projection")

    def forward(self, h, pending, ctx):
        T, ws = h.shape[0], ctx.ws
        normed = [p for p in pending if isinstance(p, NormedIncrement)]
        rest = tuple(p for p in pending if not isinstance(p, NormedIncrement))
        last = normed.pop() if normed else None
        d1, d2 = two_increments(h, rest + tuple(normed))
        xs = ws.take((T, self.d), self.env.dtype)
        # the stream with everything added, in the products' dtype
        hipops.add_rmsnorm(h, None, self.eps, out=xs, d1=d1, d2=d2, normed=last.as_arg() if last else None, plain_out=True)
        a = ws.take((T, self.dim), self.env.dtype)
        linear(xs, self.w_gate, a, ws=ws)
        g = ws.take((T, self.dim), self.env.dtype)
        hipops.gated_rows(a, ctx.token_ids, self.table, 0, g)
        y = ws.take((T, self.d), torch.float32)
        linear(g, self.w_proj, y, ws=ws)
        return (NormedIncrement(y, self.w_norm, self.mult, self.eps),)
