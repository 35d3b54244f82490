"""RMS norm: y = gain * (offset + weight) * x * rsqrt(mean(x^2) + eps), computed in float on the float residual stream.
``offset`` is 0 for a scale stored as it is and 1 for one stored around zero; ``gain`` is a constant of the layer (the
weight of a normed sublayer in the residual sum, say); both are folded into the weight once, in float, when the weights
are loaded.  ``add_normed`` is the norm of a sublayer's *output* on its way into the residual stream.

The reference computes the reduction in float, casts back and multiplies by the weight in the model's
type (src/miniserve/model.py:69-73); here the weight is applied in float too and the result is rounded once.
"""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import Norm, register_part


class RMSNorm(Norm):
    def __init__(self, prefix: str, size: int, eps: float, offset: float = 0.0, name: str = "weight", gain: float = 1.0):
        self.prefix, self.size, self.eps, self.offset, self.name = prefix, size, eps, float(offset), name
        self.gain = float(gain)

    def tensor_specs(self):
        # a scale stored around zero is drawn around zero by the random-weights mode too
        return [TensorSpec(self.prefix + self.name, (self.size,), "bias" if self.offset else "norm")]

    def load(self, get, rt):
        self.rt = rt
        self.weight = get(self.tensor_specs()[0])
        if self.offset:
            self.weight = (self.weight + self.offset).contiguous()
        if self.gain != 1.0:
            self.weight = (self.weight * self.gain).contiguous()

    def forward(self, x, delta=None, rows=None, write_back=True):
        n = x.shape[0] if rows is None else rows.numel()
        out = self.rt.empty(n, self.size)
        return ops.rms_norm(x, self.weight, self.eps, out, delta=delta, rows=rows, write_back=write_back)


    def add_normed(self, x, y, then: "RMSNorm" = None):
        """x += this norm of y, in place on the float residual stream (y: a sublayer's output, any activation type or
        float).  With ``then`` (another norm of the same width) also returns that norm of the new x, from the same
        pass over the rows."""
        if then is None:
            ops.rms_norm_add(y, self.weight, self.eps, x)
            return None
        out = self.rt.empty(x.shape[0], self.size)
        return ops.rms_norm_add(y, self.weight, self.eps, x, then.weight, then.eps, out)

    def forward_pair(self, other: "RMSNorm", x, delta=None):
        """(self's norm, ``other``'s norm) of the same rows of x (+ delta, kept in x): one pass when the two differ in
        their scales only, else two."""
        if not isinstance(other, RMSNorm) or other.size != self.size or other.eps != self.eps or \
                (delta is not None and delta.dim() != 2):
            first = self.forward(x, delta)
            return first, other.forward(x)
        n = x.shape[0]
        return ops.rms_norm_pair(x, self.weight, other.weight, self.eps, self.rt.empty(n, self.size),
                                 self.rt.empty(n, self.size), delta=delta)

    def lazy(self, x, delta=None, rows=None, write_back=True):
        """As ``forward``, for a consumer that can fold the norm into its first product: with few rows in
        bfloat16 the addend is summed into x now and the normalisation is left to that product."""
        n = x.shape[0] if rows is None else rows.numel()
        if self.rt.dtype != torch.bfloat16 or n > ops.SKINNY_MAX_ROWS or self.size % 8 or (delta is not None and not write_back):
            return self.forward(x, delta, rows, write_back)
        if delta is not None:
            ops.residual_add(x, delta)
        return linear.LazyNorm(x, self.weight, self.eps, self.rt.dtype, rows)


class LayerNorm(Norm):
    """y = weight * (x - mean x) / sqrt(mean (x - mean x)^2 + eps) (+ bias), computed in float on the float residual
    stream.  ``bias_name``: the bias tensor's name (None: the norm has none).  ``gain``: a constant the result is
    multiplied by, folded into weight and bias once, in float, when they are loaded (the scale of the logits, for a
    model's last norm).  ``forward`` also takes ``delta_scale``, a float vector the addend is multiplied by, element by
    element, on its way into x (a layer's scale)."""

    takes_delta_scale = True

    def __init__(self, prefix: str, size: int, eps: float, name: str = "weight", bias_name: str = None, gain: float = 1.0):
        self.prefix, self.size, self.eps, self.name = prefix, size, float(eps), name
        self.bias_name, self.gain = bias_name, float(gain)
        self.bias = None

    def tensor_specs(self):
        specs = [TensorSpec(self.prefix + self.name, (self.size,), "norm")]
        if self.bias_name is not None:
            specs.append(TensorSpec(self.prefix + self.bias_name, (self.size,), "bias"))
        return specs

    def load(self, get, rt):
        self.rt = rt
        specs = self.tensor_specs()
        self.weight = get(specs[0])
        self.bias = get(specs[1]) if self.bias_name is not None else None
        if self.gain != 1.0:
            self.weight = (self.weight * self.gain).contiguous()
            self.bias = (self.bias * self.gain).contiguous() if self.bias is not None else None

    def forward(self, x, delta=None, rows=None, write_back=True, delta_scale=None):
        n = x.shape[0] if rows is None else rows.numel()
        out = self.rt.empty(n, self.size)
        return ops.layer_norm(x, self.weight, self.eps, out, delta=delta, delta_scale=delta_scale, rows=rows,
                              write_back=write_back, bias=self.bias)

    def normalize_(self, x):
        """The rows of the float stream x take their own norm, in place."""
        return ops.layer_norm(x, self.weight, self.eps, x, bias=self.bias)


register_part("norm", "rms_norm", RMSNorm)
register_part("norm", "layer_norm", LayerNorm)
