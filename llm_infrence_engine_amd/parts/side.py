"""What a layer adds to the residual stream from the token itself, beside the embedding at the model's start.

``layer_scale``: a stored vector per sublayer that its result is multiplied by before the sum.

``token_side``: every layer owns a slice of ``dim`` entries of a second, narrow embedding table (``table_name``
[vocab, parts * dim], shared by the layers; layer ``part`` reads [part dim, (part + 1) dim)).  With c that slice of the
token's row:  y = proj (gelu_tanh(gate x) o c);  x <- x + y / sqrt(mean y^2 + eps) o norm, an RMS norm with a plain
weight whatever norm the model uses elsewhere.  Both maps are matrix products like any other (the first reads the
stream itself: the kernel that takes the sum still due also leaves its rows rounded to the products' type); the gate
between them is float; the norm of y and the sum into x are one kernel.
"""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import Scale, TokenInput, register_part


class LayerScale(Scale):
    def __init__(self, prefix: str, size: int, name: str):
        self.prefix, self.size, self.name = prefix, size, name

    def tensor_specs(self):
        return [TensorSpec(self.prefix + self.name, (self.size,), "norm")]

    def load(self, get, rt):
        self.rt = rt
        self.vector = get(self.tensor_specs()[0])


class TokenSide(TokenInput):
    def __init__(self, prefix: str, hidden_size: int, vocab_size: int, dim: int, part: int, parts: int, eps: float,
                 table_name: str = "side.embed", gate_name: str = "gate", proj_name: str = "proj", norm_name: str = "norm"):
        if not 0 <= part < parts or dim <= 0:
            raise ValueError(f"slice {part} of {parts} slices of {dim} entries")
        self.prefix, self.hidden_size, self.vocab_size = prefix, hidden_size, vocab_size
        self.dim, self.part, self.parts, self.eps = dim, part, parts, float(eps)
        self.table_name, self.gate_name, self.proj_name, self.norm_name = table_name, gate_name, proj_name, norm_name

    def tensor_specs(self):
        p, W, d = self.prefix, self.hidden_size, self.dim
        return [TensorSpec(self.table_name, (self.vocab_size, self.parts * d)), TensorSpec(p + self.gate_name, (d, W)),
                TensorSpec(p + self.proj_name, (W, d)), TensorSpec(p + self.norm_name, (W,), "norm")]

    def load(self, get, rt):
        self.rt = rt
        self.table, gate, proj, self.weight = (get(s) for s in self.tensor_specs())
        self.gate, self.proj = linear.prepare_weight(gate), linear.prepare_weight(proj)

    def forward(self, x, ctx, delta=None, delta_scale=None):
        N = x.shape[0]
        if self.rt.dtype == torch.float32:
            if delta is not None:
                ops.layer_norm(x, None, 0.0, None, delta=delta, delta_scale=delta_scale)
            rows = x
        else:
            rows = ops.layer_norm(x, None, 0.0, self.rt.empty(N, self.hidden_size), delta=delta, delta_scale=delta_scale)
        z = linear.linear(rows, self.gate)
        g = ops.side_gate(z, ctx.token_ids, self.table, self.part, self.rt.empty(N, self.dim))
        ops.rms_norm_add(linear.linear(g, self.proj), self.weight, self.eps, x)


register_part("scale", "layer_scale", LayerScale)
register_part("token_input", "token_side", TokenSide)
