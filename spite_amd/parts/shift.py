"""What a mixer reads instead of the normed stream itself.

``token_shift``: y[t] = x[t] + (x[t-1] - x[t]) * w, element by element, with x[t-1] the normed
stream of the request's token before t as it was before this step (zeros before the first
token).  The last normed row of a request is its state: one fp32 row per request slot, cleared
when the slot is handed out, read by the first token of the request's next portion and replaced
by the portion's last row.  The blend is fp32; the result takes the run's dtype.
"""
from __future__ import annotations

import torch

from .base import InputShift, ParamSpec, StateNeed, register
from ..csrc import hipops


@register("shift", "token_shift")
class TokenShift(InputShift):
    graph_safe = True

    def __init__(self, env, width: int):
        self.d = int(width)
        self.weight = None

    def params(self):
        return {"weight": ParamSpec((self.d,), kind="vector", init="normal")}

    def load(self, tensors):
        self.weight = tensors["weight"].float().contiguous()

    def state_need(self):
        return StateNeed((self.d,), torch.float32)

    def forward(self, x32, out, ctx, state):
        hipops.token_shift(x32, out, self.weight, state, ctx.seq_of_token, ctx.cu_seqlens, ctx.seq_slots)
