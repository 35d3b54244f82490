"""Mixers that carry a float state S [dim, vdim] per head whose rows decay by a factor of their own, made from the token.

``gated_linear_attention``: q = W_q h * dim^-1/2, k = W_k h (heads x dim), v = W_v h (heads x vdim); the decay
alpha = sigmoid(z)^(1 / tau) with z = W_a2 (W_a1 h) + bias, one number per head and key channel;
S <- diag(alpha) S + k v^T;  o = S^T q (after the write).  Every head's o is divided by its root mean square and multiplied
by a weight [vdim] shared by the heads; the heads side by side are multiplied by silu(W_g h) and projected by W_o.

``wkv``: with h' the previous token's h (zero before a request's first token), each of r, k, v, g, w reads a mix of its own,
h + (h' - h) o mu_s.  r, k, v = W_r, W_k, W_v of their mixes (heads x dim), gate = silu(W_g mix_g), decay
w = exp(-exp(W_w2 tanh(W_w1 mix_w) + w0)) per head and key channel.  o = (S + diag(u) k v^T)^T r with the bonus u [heads, dim]
for the current token alone; then S <- diag(w) S + k v^T.  Every head's o is divided by its root mean square; the heads side
by side are multiplied by a weight [heads * dim] and by the gate and projected by W_o.  State: h of the last token and S.

States, decays, their logarithms and exponentials and the read-outs' norms are float in every mode; the decays' inputs
leave their products as float."""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import Mixer, StateNeed, register_part
from .delta import _rows


class GatedLinearAttention(Mixer):
    graph_safe = True      # its kernels walk the requests from the step's device tensors

    def __init__(self, prefix: str, position, hidden_size: int, heads: int, dim: int, vdim: int, tau: float, eps: float,
                 decay_rank: int, out_scale: float = 1.0):
        if decay_rank <= 0:
            raise ValueError("the decay's low-rank map needs its rank")
        if not tau > 0:
            raise ValueError("tau must be positive")
        if dim > 256:
            raise ValueError(f"key size {dim} is not supported: the kernel holds a column of the state in registers, up to 256 rows")
        self.prefix, self.hidden_size = prefix, hidden_size
        self.heads, self.dim, self.vdim, self.tau, self.eps = heads, dim, vdim, float(tau), float(eps)
        self.decay_rank, self.out_scale = int(decay_rank), float(out_scale)
        self.qk, self.vw = heads * dim, heads * vdim

    def tensor_specs(self):
        p, W = self.prefix, self.hidden_size
        return [TensorSpec(p + "q", (self.qk, W)), TensorSpec(p + "k", (self.qk, W)), TensorSpec(p + "v", (self.vw, W)),
                TensorSpec(p + "g", (self.vw, W)), TensorSpec(p + "o", (W, self.vw)),
                TensorSpec(p + "norm", (self.vdim,), "norm"),
                TensorSpec(p + "a1", (self.decay_rank, W)), TensorSpec(p + "a2", (self.qk, self.decay_rank)),
                TensorSpec(p + "a2.b", (self.qk,), "bias")]

    def load(self, get, rt):
        self.rt = rt
        t = {s.name[len(self.prefix):]: get(s) for s in self.tensor_specs()}
        # one product for everything that reads h: q | k | v | g | a1
        self.w_in = linear.prepare_weight(torch.cat([t["q"], t["k"], t["v"], t["g"], t["a1"]], dim=0))
        self.w_a2 = linear.prepare_weight(t["a2"])
        self.w_o = linear.prepare_weight(t["o"])
        self.a_bias, self.norm_w = t["a2.b"], t["norm"]

    def state_need(self):
        return StateNeed((self.heads, self.dim, self.vdim), torch.float32)

    def forward(self, h, ctx, kv, state):
        return self.forward_residual(h, ctx, kv, state, None)

    def forward_residual(self, h, ctx, kv, state, x):
        S = state.slots
        N = ctx.num_tokens
        qk, vw = self.qk, self.vw
        g_at, a_at = 2 * qk + vw, 2 * qk + 2 * vw
        proj = linear.linear(h, self.w_in)
        z = linear.linear(_rows(proj, a_at, a_at + self.decay_rank), self.w_a2, out_dtype=torch.float32)
        o = self.rt.empty(N, vw, dtype=torch.float32)
        ops.decay_recurrence(proj[:, :qk], proj[:, qk:2 * qk], proj[:, 2 * qk:g_at], z, self.a_bias, S, ctx, o, self.heads,
                             self.dim, self.vdim, ops.DECAY_SIGMOID_ROOT, tau=self.tau, q_scale=self.dim ** -0.5)
        y = ops.gated_head_norm(o, self.norm_w, proj[:, g_at:a_at], self.rt.empty(N, vw), self.heads, self.vdim, self.eps,
                                "silu", scale=self.out_scale)
        return linear.linear_residual(y, self.w_o, None, x)


class WKV(Mixer):
    graph_safe = True

    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, prefix: str, position, hidden_size: int, heads: int, dim: int, eps: float, decay_rank: int):
        if decay_rank <= 0:
            raise ValueError("the decay's low-rank map needs its rank")
        if dim > 256:
            raise ValueError(f"key size {dim} is not supported: the kernel holds a column of the state in registers, up to 256 rows")
        self.prefix, self.hidden_size, self.heads, self.dim, self.eps = prefix, hidden_size, heads, dim, float(eps)
        self.decay_rank = int(decay_rank)
        self.inner = heads * dim

    def tensor_specs(self):
        p, W, I = self.prefix, self.hidden_size, self.inner
        specs = [TensorSpec(p + "mu." + s, (W,), "bias") for s in self.MIXES]
        specs += [TensorSpec(p + s, (I, W)) for s in ("r", "k", "v", "g")]
        specs += [TensorSpec(p + "w1", (self.decay_rank, W)), TensorSpec(p + "w2", (I, self.decay_rank)),
                  TensorSpec(p + "w0", (I,), "bias"), TensorSpec(p + "u", (self.heads, self.dim), "bias"),
                  TensorSpec(p + "norm", (I,), "norm"), TensorSpec(p + "o", (W, I))]
        return specs

    def load(self, get, rt):
        self.rt = rt
        t = {s.name[len(self.prefix):]: get(s) for s in self.tensor_specs()}
        self.mu = torch.stack([t["mu." + s] for s in self.MIXES]).contiguous()
        self.w_r, self.w_k, self.w_v, self.w_g = (linear.prepare_weight(t[s]) for s in ("r", "k", "v", "g"))
        self.w_w1, self.w_w2, self.w_o = (linear.prepare_weight(t[s]) for s in ("w1", "w2", "o"))
        self.w0, self.u, self.norm_w = t["w0"], t["u"].reshape(-1).contiguous(), t["norm"]

    def state_need(self):
        return (StateNeed((1, self.hidden_size), None), StateNeed((self.heads, self.dim, self.dim), torch.float32))

    def forward(self, h, ctx, kv, state):
        return self.forward_residual(h, ctx, kv, state, None)

    def forward_residual(self, h, ctx, kv, state, x):
        last, S = state.slots
        N, I = ctx.num_tokens, self.inner
        mixes = ops.token_shift(h, self.mu, last, ctx, self.rt.empty(len(self.MIXES), N, self.hidden_size))
        r, k, v, g = (linear.linear(mixes[i], w) for i, w in enumerate((self.w_r, self.w_k, self.w_v, self.w_g)))
        lw = ops.tanh_(linear.linear(mixes[4], self.w_w1))
        z = linear.linear(lw, self.w_w2, out_dtype=torch.float32)
        o = self.rt.empty(N, I, dtype=torch.float32)
        ops.decay_recurrence(r, k, v, z, self.w0, S, ctx, o, self.heads, self.dim, self.dim, ops.DECAY_DOUBLE_EXP, bonus=self.u)
        y = ops.gated_head_norm(o, self.norm_w, g, self.rt.empty(N, I), self.heads, self.dim, self.eps, "silu")
        return linear.linear_residual(y, self.w_o, None, x)


register_part("mixer", "gated_linear_attention", GatedLinearAttention)
register_part("mixer", "wkv", WKV)
