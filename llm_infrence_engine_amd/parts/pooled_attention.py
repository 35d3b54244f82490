"""Grouped-query attention over a sliding window of tokens and, beside it, one pooled key and value for every whole
block of older tokens.

A token at position i sees the tokens j with 0 <= i - j < ``size`` and block b (the tokens b P .. b P + P - 1, P =
``pool``) once b P + P - 1 <= i - size; a block's key is the mean of its keys as the cache holds them, its value the
mean of its values; both kinds share one softmax.  The position encoding (``rotary_pairs``) turns the first entries of
the q and k heads; with ``rotate_values`` every value is turned by its own position over its whole size before it is
cached (pairs of neighbours, pair m by position * value_theta^(-2m/value_dim)) and every head's result is turned back
by the query's position.  Scores, softmax, angles and the means are float.

Cache: two needs.  Keys and values per token, kept for the last max(size, pool) tokens (the window, and the block that
is being filled); and one pooled key and value per block, kept for good, in pages of their own that hold an entry for
every ``pool`` tokens."""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import CacheNeed, Mixer, PageTensor, register_part

_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o"}


class PooledWindowAttention(Mixer):
    graph_safe = True

    def __init__(self, prefix: str, position, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 value_dim: int, scale: float, size: int, pool: int, rotate_values: bool = True,
                 value_theta: float = 10000.0, names=None):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads cannot share {num_kv_heads} key/value heads")
        if not (0 < head_dim <= 256 and 0 < value_dim <= 256) or head_dim % 2 or value_dim % 2:
            raise ValueError("key and value sizes are even and at most 256")
        if size <= 0 or pool <= 0:
            raise ValueError("the window and the pooled blocks hold at least one token")
        if position is not None and not hasattr(position, "inv_freq") and not hasattr(position, "dims"):
            raise ValueError("this mixer turns pairs of neighbours: it takes the position encoding 'rotary_pairs' or none")
        self.prefix, self.position = prefix, position
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.value_dim, self.scale = head_dim, value_dim, float(scale)
        self.size, self.pool = int(size), int(pool)
        self.rotate_values, self.value_theta = bool(rotate_values), float(value_theta)
        self.names = dict(_NAMES, **dict(names or {}))

    def tensor_specs(self):
        p, W, d, dv = self.prefix, self.hidden_size, self.head_dim, self.value_dim
        return [TensorSpec(p + self.names["q"], (self.num_heads * d, W)), TensorSpec(p + self.names["k"], (self.num_kv_heads * d, W)),
                TensorSpec(p + self.names["v"], (self.num_kv_heads * dv, W)), TensorSpec(p + self.names["o"], (W, self.num_heads * dv))]

    def load(self, get, rt):
        self.rt = rt
        q, k, v, o = (get(s) for s in self.tensor_specs())
        self.w_qkv = linear.prepare_weight(torch.cat([q, k, v], dim=0))
        self.w_o = linear.prepare_weight(o)
        if self.position is not None:
            self.position.load(get, rt)
            self.rot_dims, self.inv_freq = self.position.dims, self.position.inv_freq
        else:
            self.rot_dims, self.inv_freq = 0, torch.zeros(0, dtype=torch.float32, device=rt.device)
        m = torch.arange(0, self.value_dim, 2, dtype=torch.float64)
        f = self.value_theta ** (-m / self.value_dim) if self.rotate_values else torch.zeros_like(m)
        self.inv_freq_v = f.to(torch.float32).to(rt.device)

    def cache_need(self):
        # in bfloat16 the matrix-core kernel reads value pages (of tokens and of blocks) as an operand as they lie,
        # transposed, which it can for values of the keys' size in pages of a multiple of 16 tokens
        flip = dict(transpose_at=16, transpose_in=torch.bfloat16) if self.value_dim == self.head_dim else {}
        tensors = (PageTensor("k", self.num_kv_heads, self.head_dim), PageTensor("v", self.num_kv_heads, self.value_dim, **flip))
        return (CacheNeed(tensors, window=max(self.size, self.pool)), CacheNeed(tensors, stride=self.pool))

    def forward(self, h, ctx, kv, state):
        if kv is None or len(kv.more) != 1:
            raise RuntimeError("this attention needs the view of its token pages with the view of its pooled pages in it")
        pooled = kv.more[0]
        nh, nkv, d, dv = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        qkv = linear.linear(h, self.w_qkv)
        ops.pairs_rotate_store(qkv, nh, nkv, d, dv, self.rot_dims, ctx.positions, self.inv_freq, self.inv_freq_v, kv)
        if kv.store:
            ops.pool_store(kv, pooled, ctx, self.pool)
        out = self.rt.empty(ctx.num_tokens, nh * dv)
        turn_back = None
        if self.rotate_values and qkv.dtype == torch.bfloat16 and kv.transposed.get("v"):
            # cosines and sines of the step's positions: worked out by the first layer that comes here, shared by the others
            key = ("rotary_pairs", dv, self.value_theta)
            turn_back = ctx.shared.get(key)
            if turn_back is None:
                turn_back = ctx.shared[key] = ops.rope_table(ctx.positions, self.inv_freq_v)
        ops.pooled_attention(qkv, kv, pooled, ctx, out, nh, self.scale, self.size, self.pool,
                             self.inv_freq_v if self.rotate_values else None, turn_back)
        return linear.linear(out, self.w_o)


register_part("mixer", "pooled_window_attention", PooledWindowAttention)
