"""Dense gated feed-forward: down(silu(gate(x)) * up(x)), no biases (src/miniserve/model.py:155-165).
Gate and up are one packed matrix product (rows interleaved so that the activation can be the product's
epilogue); the activation is float."""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import FeedForward, register_part


class SwiGLU(FeedForward):
    accepts_lazy_norm = True

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int):
        self.prefix, self.hidden_size, self.intermediate_size = prefix, hidden_size, intermediate_size

    def tensor_specs(self):
        p, H, I = self.prefix, self.hidden_size, self.intermediate_size
        return [TensorSpec(p + "gate_proj.weight", (I, H)), TensorSpec(p + "up_proj.weight", (I, H)),
                TensorSpec(p + "down_proj.weight", (H, I))]

    def load(self, get, rt):
        self.rt = rt
        g, u, d = (get(s) for s in self.tensor_specs())
        self.w_gate_up = linear.interleave_rows(g, u)
        self.w_down = linear.prepare_weight(d)

    def forward(self, h, ctx):
        return self.forward_residual(h, ctx, None)

    def forward_residual(self, h, ctx, x):
        return linear.linear_residual(linear.linear_swiglu(h, self.w_gate_up), self.w_down, None, x)


class DenseAct(FeedForward):
    """down(act(up(x))), no biases.  ``activation``: "xielu", with two learned numbers (p, q) in the tensor ``act``:
    z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2; or "gelu", the exact one,
    z/2 (1 + erf(z / sqrt 2)), which has no tensor."""

    ACTIVATIONS = ("xielu", "gelu")

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, activation: str = "xielu"):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"no activation {activation!r}; there are {', '.join(self.ACTIVATIONS)}")
        self.prefix, self.hidden_size, self.intermediate_size, self.activation = prefix, hidden_size, intermediate_size, activation

    def tensor_specs(self):
        p, H, I = self.prefix, self.hidden_size, self.intermediate_size
        specs = [TensorSpec(p + "up", (I, H)), TensorSpec(p + "down", (H, I))]
        return specs + ([TensorSpec(p + "act", (2,), "bias")] if self.activation == "xielu" else [])

    def load(self, get, rt):
        self.rt = rt
        up, down, *act = (get(s) for s in self.tensor_specs())
        self.w_up, self.w_down, self.act = linear.prepare_weight(up), linear.prepare_weight(down), (act[0] if act else None)

    def forward(self, h, ctx):
        return self.forward_residual(h, ctx, None)

    def forward_residual(self, h, ctx, x):
        u = linear.linear(h, self.w_up)
        u = ops.xielu(u, self.act, torch.empty_like(u)) if self.activation == "xielu" else ops.gelu(u, torch.empty_like(u))
        return linear.linear_residual(u, self.w_down, None, x)


class ClampedGLU(FeedForward):
    """down(g * sigmoid(alpha g) * (u + 1)) with g = min(gate(x), limit) and u = clamp(up(x), -limit, limit); no biases.
    Gate and up are one packed product (rows interleaved); clamps and activation are float."""

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, limit: float, alpha: float = 1.702,
                 gate_name: str = "gate", up_name: str = "up", down_name: str = "down"):
        self.prefix, self.hidden_size, self.intermediate_size = prefix, hidden_size, intermediate_size
        self.limit, self.alpha = float(limit), float(alpha)
        self.gate_name, self.up_name, self.down_name = gate_name, up_name, down_name

    def tensor_specs(self):
        p, H, I = self.prefix, self.hidden_size, self.intermediate_size
        return [TensorSpec(p + self.gate_name, (I, H)), TensorSpec(p + self.up_name, (I, H)), TensorSpec(p + self.down_name, (H, I))]

    def load(self, get, rt):
        self.rt = rt
        g, u, d = (get(s) for s in self.tensor_specs())
        self.w_gate_up = linear.interleave_rows(g, u)
        self.w_down = linear.prepare_weight(d)

    def forward(self, h, ctx):
        gu = linear.linear(h, self.w_gate_up)
        act = ops.clamped_glu(gu, self.rt.empty(gu.shape[0], self.intermediate_size), self.limit, self.alpha)
        return linear.linear(act, self.w_down)


class GatedGLU(FeedForward):
    """down(act(gate(x)) * up(x)), no biases, with ``activation`` "gelu_tanh": z/2 (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))),
    or "silu" (the gated feed-forward above, under other tensor names).  Gate and up are one packed product (rows
    interleaved); the activation is float."""

    ACTIVATIONS = ("gelu_tanh", "silu")

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, activation: str = "gelu_tanh",
                 gate_name: str = "gate", up_name: str = "up", down_name: str = "down"):
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"no activation {activation!r}; there are {', '.join(self.ACTIVATIONS)}")
        self.prefix, self.hidden_size, self.intermediate_size, self.activation = prefix, hidden_size, intermediate_size, activation
        self.gate_name, self.up_name, self.down_name = gate_name, up_name, down_name

    def tensor_specs(self):
        p, H, I = self.prefix, self.hidden_size, self.intermediate_size
        return [TensorSpec(p + self.gate_name, (I, H)), TensorSpec(p + self.up_name, (I, H)), TensorSpec(p + self.down_name, (H, I))]

    def load(self, get, rt):
        self.rt = rt
        g, u, d = (get(s) for s in self.tensor_specs())
        self.w_gate_up = linear.interleave_rows(g, u)
        self.w_down = linear.prepare_weight(d)

    def forward(self, h, ctx):
        return self.forward_residual(h, ctx, None)

    def forward_residual(self, h, ctx, x):
        if self.activation == "silu":
            act = linear.linear_swiglu(h, self.w_gate_up)
        else:
            act = None
            if h.dtype == torch.bfloat16 and h.shape[0] > ops.SKINNY_MAX_ROWS and ops.gemm_tiled_pays(h, self.w_gate_up):
                try:        # many rows: the activation is the product's epilogue
                    act = ops.gemm_tiled(h, self.w_gate_up, ops.EPI_GEGLU)
                except ops.UnsupportedShape:
                    act = None
            if act is None:
                gu = linear.linear(h, self.w_gate_up)
                act = ops.gelu_tanh_glu(gu, self.rt.empty(gu.shape[0], self.intermediate_size))
        return linear.linear_residual(act, self.w_down, None, x)


register_part("feed_forward", "swiglu", SwiGLU)
register_part("feed_forward", "gated_glu", GatedGLU)
register_part("feed_forward", "clamped_glu", ClampedGLU)
register_part("feed_forward", "dense_act", DenseAct)
