"""Grouped-query attention over the paged cache.

q, k, v projections (one packed matrix product), position encoding fused with the cache store, causal
attention read in place from the pages, output projection.  Query head h uses key/value head
h // (num_heads // num_kv_heads) (src/miniserve/model.py:137-139).  Scores, softmax and the weighted
sum are float.  ``window`` limits a query to the last ``window`` keys (None: all).  ``value_dim``: values of another
size than queries and keys.  ``sink``: a learned number per query head (tensor ``sink`` [heads]) whose exponential joins
the softmax's denominator; it has no key and no value and is not scaled; ``sink="zero"``: the same with the constant 0 for
every head and no tensor (one is added to the denominator).  ``softcap`` c: a scaled score s becomes c tanh(s / c).
``slope_base`` b: head h of H takes slope_h (i - j) off the score of key j for query i, slope_h = 2^(-b (h + 1) / H) (after the
cap).  ``gate``: a projection [heads, hidden] (tensor "gate") whose sigmoid multiplies every head's result, one number per
token and head, before the output projection; it rides on the packed q/k/v product.  ``out_scale`` multiplies the heads'
results.  ``names``: the tensors' names after the prefix, {"q", "k", "v", "o", "sink", "gate"} -> name; biases are the weight's
name with ".bias" for ".weight", or the weight's name followed by ``bias_suffix``.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import CacheNeed, KVNeed, Mixer, PageTensor, register_part

_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight", "sink": "sink",
          "gate": "gate"}


class GQAttention(Mixer):
    accepts_lazy_norm = True

    def __init__(self, prefix: str, position, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 scale: float, qkv_bias: bool = True, out_bias: bool = False, window: Optional[int] = None,
                 value_dim: Optional[int] = None, sink=False, names=None, softcap: Optional[float] = None,
                 slope_base: Optional[float] = None, gate: bool = False, out_scale: float = 1.0,
                 bias_suffix: Optional[str] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads cannot share {num_kv_heads} key/value heads")
        if not 0 < head_dim <= 256:
            raise ValueError(f"head_dim {head_dim} is not supported: the attention kernels take sizes up to 256")
        if window is not None and window <= 0:
            raise ValueError("window must be positive")
        self.prefix, self.position = prefix, position
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.scale, self.qkv_bias, self.out_bias, self.window = float(scale), qkv_bias, out_bias, window
        self.value_dim = head_dim if value_dim is None else int(value_dim)
        if not 0 < self.value_dim <= 256:
            raise ValueError(f"value size {self.value_dim} is not supported: the attention kernels take up to 256")
        if self.value_dim != head_dim and not getattr(position, "takes_value_dim", False):
            raise ValueError("values of another size than keys need a position encoding that stores them "
                             "(one with takes_value_dim)")
        if sink not in (False, True, "zero"):
            raise ValueError(f"sink is False, True (a learned number per head) or 'zero', got {sink!r}")
        self.sink = sink is True
        self.zero_sink = sink == "zero"
        if softcap is not None and not softcap > 0:
            raise ValueError("softcap must be positive")
        self.softcap = float(softcap) if softcap is not None else 0.0
        self.slope_base = float(slope_base) if slope_base is not None else None
        self.gate, self.out_scale, self.bias_suffix = bool(gate), float(out_scale), bias_suffix
        self.names = dict(_NAMES, **dict(names or {}))
        self.slopes = self.w_gate_rows = None

    def _bias_name(self, which: str) -> str:
        name = self.names[which]
        if self.bias_suffix is not None:
            return name + self.bias_suffix
        return name[:-len(".weight")] + ".bias" if name.endswith(".weight") else name + ".bias"

    # ---- weights
    def tensor_specs(self):
        p, H, d, dv = self.prefix, self.hidden_size, self.head_dim, self.value_dim
        specs = []
        for which, rows in (("q", self.num_heads * d), ("k", self.num_kv_heads * d), ("v", self.num_kv_heads * dv)):
            specs.append(TensorSpec(p + self.names[which], (rows, H)))
            if self.qkv_bias:
                specs.append(TensorSpec(p + self._bias_name(which), (rows,), "bias"))
        specs.append(TensorSpec(p + self.names["o"], (H, self.num_heads * dv)))
        if self.out_bias:
            specs.append(TensorSpec(p + self._bias_name("o"), (H,), "bias"))
        if self.sink:
            specs.append(TensorSpec(p + self.names["sink"], (self.num_heads,), "bias"))
        if self.gate:
            specs.append(TensorSpec(p + self.names["gate"], (self.num_heads, H)))
        if self.position is not None:
            specs += self.position.tensor_specs()
        return specs

    def load(self, get, rt):
        self.rt = rt
        by_name = {s.name: s for s in GQAttention.tensor_specs(self)}
        p = self.prefix
        w = [get(by_name[p + self.names[n]]) for n in ("q", "k", "v")]
        if self.gate:       # the gate's rows ride on the packed product, after q, k and v; rows of zeros make the
            w.append(get(by_name[p + self.names["gate"]]))      # product's rows a multiple of 16 bytes, as the matrix-core attention reads q
            pad = (-sum(t.shape[0] for t in w)) % 8
            if pad:
                w.append(torch.zeros(pad, self.hidden_size, dtype=w[0].dtype, device=w[0].device))
        self.w_qkv = linear.prepare_weight(torch.cat(w, dim=0))
        self.b_qkv = None
        if self.qkv_bias:
            b = [get(by_name[p + self._bias_name(n)]) for n in ("q", "k", "v")]
            if self.gate:
                b.append(torch.zeros(self.w_qkv.shape[0] - sum(t.numel() for t in b), dtype=b[0].dtype, device=b[0].device))
            self.b_qkv = torch.cat(b).contiguous()
        self.w_o = linear.prepare_weight(get(by_name[p + self.names["o"]]))
        self.b_o = get(by_name[p + self._bias_name("o")]) if self.out_bias else None
        self.sink_w = get(by_name[p + self.names["sink"]]) if self.sink else None
        if self.zero_sink:
            self.sink_w = torch.zeros(self.num_heads, dtype=torch.float32, device=rt.device)
        if self.slope_base is not None:
            H = self.num_heads
            self.slopes = torch.tensor([2.0 ** (-self.slope_base * (h + 1) / H) for h in range(H)], dtype=torch.float64) \
                .to(torch.float32).to(rt.device)
        if self.position is not None:
            self.position.load(get, rt)

    # ---- cache
    def cache_need(self):
        # in bfloat16 the matrix-core attention reads value pages as an operand as they lie, transposed, which it
        # can for pages of a multiple of 16 tokens
        if self.value_dim == self.head_dim:
            return KVNeed(self.num_kv_heads, self.head_dim, self.window, transpose_values_at=16,
                          transpose_values_in=torch.bfloat16)
        return CacheNeed((PageTensor("k", self.num_kv_heads, self.head_dim),
                          PageTensor("v", self.num_kv_heads, self.value_dim)), self.window)

    # ---- step
    def forward(self, h, ctx, kv, state):
        return self.forward_residual(h, ctx, kv, state, None)

    def forward_residual(self, h, ctx, kv, state, x):
        if kv is None:
            raise RuntimeError("attention needs a key/value cache view")
        nh, nkv, d, dv = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        if self.gate:
            return self._forward_gated(h, ctx, kv, x)
        q = None
        if self.position is not None and dv == d:
            q = self.position.project_encode_store(h, self.w_qkv, self.b_qkv, nh, nkv, d, ctx, kv)
        if q is None:
            # [N, (nh + 2 nkv) d]: attention reads its q part.  A library product has no bias epilogue; a position
            # encoding that can add the bias on its way saves a pass over the projection.
            late_bias = (self.b_qkv is not None and getattr(self.position, "adds_bias", False)
                         and linear.goes_to_library(h, self.w_qkv))
            q = linear.linear(h, self.w_qkv, bias=None if late_bias else self.b_qkv)
            if late_bias:
                self.position.encode_and_store(q, nh, nkv, d, ctx, kv, bias=self.b_qkv)
            elif dv != d:
                self.position.encode_and_store(q, nh, nkv, d, ctx, kv, value_dim=dv)
            elif self.position is not None:
                self.position.encode_and_store(q, nh, nkv, d, ctx, kv)
            elif kv.store:
                ops.rope_store(q, nh, nkv, d, 0, None, None, kv.slot_mapping, kv.k_pages, kv.v_pages, kv.v_transposed)
        out = self.rt.empty(ctx.num_tokens, nh * dv)
        ops.paged_attention(q, kv, ctx, out, nh, self.scale, self.window, self.sink_w, self.softcap, self.slopes, None,
                            self.out_scale)
        return linear.linear_residual(out, self.w_o, self.b_o, x)

    def _forward_gated(self, h, ctx, kv, x):
        """With an output gate: one product for q, k, v and the gate's numbers; the position encoding works on the first
        columns, the attention kernel reads the last ones."""
        nh, nkv, d, dv = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        width = (nh + nkv) * d + nkv * dv
        proj = linear.linear(h, self.w_qkv, bias=self.b_qkv)
        qkv = proj[:, :width]
        if self.position is None:
            if kv.store:
                ops.qk_norm_store(qkv, nh, nkv, d, dv, None, None, 0.0, slot_mapping=kv.slot_mapping, k_pages=kv.k_pages,
                                  v_pages=kv.v_pages, v_transposed=kv.v_transposed)
        elif dv != d or getattr(self.position, "takes_value_dim", False):
            self.position.encode_and_store(qkv, nh, nkv, d, ctx, kv, value_dim=dv)
        else:
            self.position.encode_and_store(qkv, nh, nkv, d, ctx, kv)
        out = self.rt.empty(ctx.num_tokens, nh * dv)
        ops.paged_attention(qkv, kv, ctx, out, nh, self.scale, self.window, self.sink_w, self.softcap, self.slopes,
                            proj[:, width:width + nh], self.out_scale)
        return linear.linear_residual(out, self.w_o, self.b_o, x)


register_part("mixer", "gqa_attention", GQAttention)
