"""minGRU: a gated recurrence per channel whose gates read only the current token, without a cache of keys.

h -> [pz | px | pg] (``width`` each) by one packed product;  z = sigmoid(pz + bz);  u = px + bx;  the candidate is
c = u + 1/2 where u >= 0 and sigmoid(u) below;  S_t = (1 - z) S_(t-1) + z c channel by channel, from S = 0;
out = W_o (S_t * silu(pg)).  State per request: S [width], float; gates, candidate and the read-out's gate are float in
every mode (the biases join in float inside the recurrence's kernel, not in the product)."""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import Mixer, StateNeed, register_part


class MinGRU(Mixer):
    graph_safe = True      # its kernel walks the requests from the step's device tensors

    def __init__(self, prefix: str, position, hidden_size: int, width: int):
        if width <= 0:
            raise ValueError("width must be positive")
        self.prefix, self.hidden_size, self.width = prefix, hidden_size, width

    def tensor_specs(self):
        p, W, C = self.prefix, self.hidden_size, self.width
        return [TensorSpec(p + "z", (C, W)), TensorSpec(p + "z.b", (C,), "bias"), TensorSpec(p + "x", (C, W)),
                TensorSpec(p + "x.b", (C,), "bias"), TensorSpec(p + "g", (C, W)), TensorSpec(p + "o", (W, C))]

    def load(self, get, rt):
        self.rt = rt
        t = {s.name[len(self.prefix):]: get(s) for s in self.tensor_specs()}
        self.w_zxg = linear.prepare_weight(torch.cat([t["z"], t["x"], t["g"]], dim=0))
        self.b_z, self.b_x = t["z.b"], t["x.b"]
        self.w_o = linear.prepare_weight(t["o"])

    def state_need(self):
        return StateNeed((self.width,), torch.float32)

    def forward(self, h, ctx, kv, state):
        zxg = linear.linear(h, self.w_zxg)
        y = ops.mingru_scan(zxg, self.b_z, self.b_x, state.slots, ctx, self.rt.empty(ctx.num_tokens, self.width))
        return linear.linear(y, self.w_o)


register_part("mixer", "mingru", MinGRU)
