"""Rotary position encoding with half-split pairing.

inv_freq[j] = theta^(-2j/rotary_dim); the pair (j, j + rotary_dim/2) of every q and k head turns by
position * inv_freq[j] (src/miniserve/model.py:83-98).  Angles, sines and cosines are float in every
mode; the frequencies are derived in double on the host and rounded once.  The rotation is fused with
the store of k and v into the cache pages.
"""
from __future__ import annotations

import math

import torch

from ..kernels import linear, ops
from .base import PositionEncoding, register_part


class RotaryHalf(PositionEncoding):
    adds_bias = True   # encode_and_store takes ``bias`` and adds it to q, k, v before rotating and storing

    def __init__(self, prefix: str, head_dim: int, rotary_dim: int, theta: float):
        if rotary_dim % 2 or not 0 < rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {rotary_dim} must be even and within head_dim {head_dim}")
        self.head_dim, self.rotary_dim, self.theta = head_dim, rotary_dim, float(theta)

    def load(self, get, rt):
        self.rt = rt
        j = torch.arange(0, self.rotary_dim, 2, dtype=torch.float64)
        self.inv_freq = (1.0 / (self.theta ** (j / self.rotary_dim))).to(torch.float32).to(rt.device)

    def project_encode_store(self, h, w_qkv, bias, num_heads, num_kv_heads, head_dim, ctx, kv):
        if (kv is not None and kv.store
                and ops.gemm_tiled_qkv_pays(h, w_qkv, head_dim, self.rotary_dim, kv.k_pages)):
            # a portion of a prompt: rotation and cache store are the product's epilogue; the cosines and sines of
            # the step's positions are worked out by the first layer that comes here and shared by the others
            key = ("rotary_half", self.rotary_dim, self.theta)
            table = ctx.shared.get(key)
            if table is None:
                table = ctx.shared[key] = ops.rope_table(ctx.positions, self.inv_freq)
            return ops.gemm_tiled_qkv(h, w_qkv, bias, num_heads, num_kv_heads, head_dim, table, kv.slot_mapping,
                                      kv.k_pages, kv.v_pages, kv.v_transposed)
        if not (isinstance(h, linear.LazyNorm) and h.rows is None and kv is not None and kv.store
                and ops.qkv_rope_store_ok(h.x, w_qkv, head_dim, self.rotary_dim) and ops.qkv_rope_store_pays(h.x, w_qkv)):
            return None
        return ops.qkv_rope_store(h.x, h.weight, h.eps, w_qkv, bias, num_heads, num_kv_heads, head_dim, ctx.positions,
                                  self.inv_freq, kv.slot_mapping, kv.k_pages, kv.v_pages, kv.v_transposed)

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, kv, bias=None):
        store = kv is not None and kv.store
        ops.rope_store(qkv, num_heads, num_kv_heads, head_dim, self.rotary_dim, ctx.positions, self.inv_freq,
                       kv.slot_mapping if store else None, kv.k_pages if store else None,
                       kv.v_pages if store else None, store and kv.v_transposed, bias)


class NoPosition(PositionEncoding):
    """No encoding: k and v are stored as they are."""

    def __init__(self, prefix: str = ""):
        pass

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, kv):
        if kv is not None and kv.store:
            ops.rope_store(qkv, num_heads, num_kv_heads, head_dim, 0, None, None, kv.slot_mapping, kv.k_pages,
                           kv.v_pages, kv.v_transposed)


class RotaryPairs(PositionEncoding):
    """Rotary encoding with neighbouring entries paired: of a vector's first ``dims`` entries, entry 2i and entry
    2i + 1 turn by position * theta^(-2i/dims); the rest pass unchanged.  It turns whatever slice of a vector its
    mixer hands it (``rotate``); angles, sines and cosines are float."""

    def __init__(self, prefix: str, width: int, dims: int, theta: float):
        if dims % 2 or not 0 <= dims <= width:
            raise ValueError(f"{dims} rotated entries must be even and within the vector's width {width}")
        self.width, self.dims, self.theta = width, dims, float(theta)

    def load(self, get, rt):
        self.rt = rt
        i = torch.arange(0, self.dims, 2, dtype=torch.float64)
        self.inv_freq = (self.theta ** (-i / max(1, self.dims))).to(torch.float32).to(rt.device)

    def rotate(self, src, dst, ctx):
        """dst[n, h] = src[n, h] turned by the position of token n; [N, heads, width] views, dst may be src."""
        return ops.rotary_pairs(src, dst, ctx.positions, self.inv_freq)


class QKNormTemperature(PositionEncoding):
    """Heads that are normalised instead of rotated.  Every query and key head passes an RMS norm with a weight of
    its own kind (``q_norm`` / ``k_norm`` [head_dim], shared by the heads; ``qk_norm`` False: no norm), and the position
    enters through a query temperature alone: q of the token at position p is multiplied by
    1 + coef * ln(floor((p + 1) / every) + 1) (``coef`` 0 or None: no temperature).  Keys and values may differ in size.
    Norm, logarithm and temperature are float; one kernel also stores k and v into the pages."""

    takes_value_dim = True

    def __init__(self, prefix: str, head_dim: int, eps: float, qk_norm: bool = True, coef: float = 0.0, every: int = 1,
                 q_norm_name: str = "q.norm", k_norm_name: str = "k.norm"):
        if coef and every <= 0:
            raise ValueError("the query temperature's period must be positive")
        self.prefix, self.head_dim, self.eps, self.qk_norm = prefix, head_dim, float(eps), bool(qk_norm)
        self.coef, self.every = float(coef or 0.0), int(every)
        self.q_norm_name, self.k_norm_name = q_norm_name, k_norm_name
        self.q_weight = self.k_weight = None

    def tensor_specs(self):
        if not self.qk_norm:
            return []
        from ..weights.spec import TensorSpec

        return [TensorSpec(self.prefix + self.q_norm_name, (self.head_dim,), "norm"),
                TensorSpec(self.prefix + self.k_norm_name, (self.head_dim,), "norm")]

    def load(self, get, rt):
        self.rt = rt
        if self.qk_norm:
            self.q_weight, self.k_weight = (get(s) for s in self.tensor_specs())

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, kv, value_dim=None):
        store = kv is not None and kv.store
        ops.qk_norm_store(qkv, num_heads, num_kv_heads, head_dim, head_dim if value_dim is None else value_dim,
                          self.q_weight, self.k_weight, self.eps, ctx.positions, self.coef, self.every,
                          kv.slot_mapping if store else None, kv.k_pages if store else None,
                          kv.v_pages if store else None, bool(store and kv.v_transposed))


def scaled_frequencies(dims: int, base: float, scaling=None) -> torch.Tensor:
    """f_i = base^(-2 i / dims) for i < dims / 2, in double.  ``scaling`` {"factor", "low", "high", "original"} stretches
    the long waves: with a wavelength l = 2 pi / f below original / high, f stays; above original / low, f / factor; in
    between, with s = (original / l - low) / (high - low), the blend (1 - s) f / factor + s f."""
    i = torch.arange(0, dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / max(1, dims))
    if scaling is None:
        return f
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    if high == low:
        raise ValueError("frequency scaling needs high != low")
    wave = 2.0 * math.pi / f
    s = (original / wave - low) / (high - low)
    blended = (1.0 - s) * f / factor + s * f
    return torch.where(wave < original / high, f, torch.where(wave > original / low, f / factor, blended))


class QKNormRotaryHalf(PositionEncoding):
    """Heads that are normalised and then rotated.  Every query and key head is divided by its root mean square (eps inside
    the root) and, with ``weighted``, multiplied by a weight of its kind (``q_norm_name`` / ``k_norm_name`` [head_dim], shared
    by the heads); then, with ``dims`` > 0, entry i and entry i + dims / 2 of the head's first ``dims`` entries turn by
    position * f_i (``scaled_frequencies``); the rest pass.  Keys and values may differ in size.  Norm, angles, sines and
    cosines are float; one kernel also stores k and v into the pages."""

    takes_value_dim = True

    def __init__(self, prefix: str, head_dim: int, eps: float, weighted: bool = True, dims: int = 0, base: float = 10000.0,
                 scaling=None, q_norm_name: str = "q.norm", k_norm_name: str = "k.norm"):
        if dims % 2 or not 0 <= dims <= head_dim:
            raise ValueError(f"{dims} rotated entries must be even and within the head's {head_dim}")
        self.prefix, self.head_dim, self.eps, self.weighted = prefix, head_dim, float(eps), bool(weighted)
        self.dims, self.base = int(dims), float(base)
        self.scaling = dict(scaling) if scaling is not None else None
        self.q_norm_name, self.k_norm_name = q_norm_name, k_norm_name
        self.q_weight = self.k_weight = self.inv_freq = None

    def tensor_specs(self):
        if not self.weighted:
            return []
        from ..weights.spec import TensorSpec

        return [TensorSpec(self.prefix + self.q_norm_name, (self.head_dim,), "norm"),
                TensorSpec(self.prefix + self.k_norm_name, (self.head_dim,), "norm")]

    def load(self, get, rt):
        self.rt = rt
        if self.weighted:
            self.q_weight, self.k_weight = (get(s) for s in self.tensor_specs())
        if self.dims:
            self.inv_freq = scaled_frequencies(self.dims, self.base, self.scaling).to(torch.float32).to(rt.device)

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, kv, value_dim=None):
        store = kv is not None and kv.store
        ops.qk_norm_store(qkv, num_heads, num_kv_heads, head_dim, head_dim if value_dim is None else value_dim,
                          self.q_weight, self.k_weight, self.eps, ctx.positions, 0.0, 1,
                          kv.slot_mapping if store else None, kv.k_pages if store else None,
                          kv.v_pages if store else None, bool(store and kv.v_transposed), unit_norm=True,
                          inv_freq=self.inv_freq, rot_dim=self.dims)


register_part("position", "qk_norm_rotary_half", QKNormRotaryHalf)
register_part("position", "qk_norm_temperature", QKNormTemperature)
register_part("position", "rotary_half", RotaryHalf)
register_part("position", "rotary_pairs", RotaryPairs)
register_part("position", "none", NoPosition)
