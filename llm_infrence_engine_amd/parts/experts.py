"""A feed-forward made of routed experts.

Router logits z = W_router h in float; scores s = softmax(z) over all the router's outputs; the ``top`` outputs with the
largest s + correction are chosen (``correction``: a stored vector that steers the choice and nothing else; False: there is
none) and weigh in with their s as it is.  ``scores`` "sigmoid": s is every logit's own sigmoid.  ``activation`` "swiglu":
an expert is down(silu(gate(h)) * up(h)) with a third matrix ``gate``.  ``weight_on`` "input": the weight multiplies what
the expert reads instead of what it returns, out = sum expert(s h) (both first products are linear, so the kernel applies
s to their results, in float, before the activation).  The first ``experts`` outputs are small feed-forwards down(act(up(h))) without biases; the last
``identity`` outputs are experts without tensors whose output is h itself.  ``shared_ff``: one more expert of that size
that every token runs, weighted by sigmoid(W_sg h), one number per token.

Nothing here waits for the device: the tokens' choices are grouped by expert into tiles on the device, and the experts'
products run tile by tile over a launch whose size depends on the sizes alone, so a step can be captured."""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import FeedForward, register_part


class RoutedExperts(FeedForward):
    def __init__(self, prefix: str, hidden_size: int, expert_ff: int, experts: int, top: int, identity: int = 0,
                 shared_ff: int = 0, activation: str = "gelu", scores: str = "softmax", correction: bool = True,
                 weight_on: str = "output"):
        if activation not in ("gelu", "swiglu"):
            raise ValueError(f"no activation {activation!r} for routed experts; there are 'gelu' and 'swiglu'")
        if scores not in ("softmax", "sigmoid") or weight_on not in ("output", "input"):
            raise ValueError("scores are 'softmax' or 'sigmoid'; the weight lies on the expert's 'output' or 'input'")
        if weight_on == "input" and (activation != "swiglu" or identity or shared_ff):
            raise ValueError("a weight on the expert's input comes with 'swiglu' experts alone")
        if experts <= 0 or identity < 0 or not 0 < top <= experts + identity:
            raise ValueError(f"{top} of {experts} + {identity} experts cannot be chosen")
        if experts + identity > ops.ROUTE_MAX_OUTPUTS or top > ops.ROUTE_MAX_TOP:
            raise ValueError(f"the router kernel takes up to {ops.ROUTE_MAX_OUTPUTS} outputs and a top of {ops.ROUTE_MAX_TOP}")
        self.prefix, self.hidden_size, self.expert_ff = prefix, hidden_size, expert_ff
        self.experts, self.identity, self.top, self.shared_ff = experts, identity, top, shared_ff
        self.activation, self.scores, self.has_correction, self.weight_on = activation, scores, bool(correction), weight_on

    def tensor_specs(self):
        p, W, F = self.prefix, self.hidden_size, self.expert_ff
        specs = []
        for e in range(self.experts):
            if self.activation == "swiglu":
                specs.append(TensorSpec(f"{p}e{e}.gate", (F, W)))
            specs += [TensorSpec(f"{p}e{e}.up", (F, W)), TensorSpec(f"{p}e{e}.down", (W, F))]
        n_out = self.experts + self.identity
        specs.append(TensorSpec(p + "router", (n_out, W)))
        if self.has_correction:
            specs.append(TensorSpec(p + "correction", (n_out,), "bias"))
        if self.shared_ff:
            specs += [TensorSpec(p + "shared.up", (self.shared_ff, W)), TensorSpec(p + "shared.down", (W, self.shared_ff)),
                      TensorSpec(p + "shared.sg", (1, W))]
        return specs

    def load(self, get, rt):
        self.rt = rt
        t = {s.name[len(self.prefix):]: get(s) for s in self.tensor_specs()}
        if self.activation == "swiglu":      # gate and up rows interleaved, expert by expert: [E, 2F, W]
            self.w_up = torch.stack([linear.interleave_rows(t[f"e{e}.gate"], t[f"e{e}.up"]) for e in range(self.experts)]).contiguous()
        else:
            self.w_up = torch.stack([t[f"e{e}.up"] for e in range(self.experts)]).contiguous()       # [E, F, W]
        self.w_down = torch.stack([t[f"e{e}.down"] for e in range(self.experts)]).contiguous()   # [E, W, F]
        # the router and the shared expert's gate read the same h: one product, float out
        self.w_router = linear.prepare_weight(torch.cat([t["router"]] + ([t["shared.sg"]] if self.shared_ff else []), dim=0))
        self.correction = t["correction"] if self.has_correction else None
        if self.shared_ff:
            self.w_shared_up, self.w_shared_down = linear.prepare_weight(t["shared.up"]), linear.prepare_weight(t["shared.down"])

    def forward(self, h, ctx):
        N, W, E = h.shape[0], self.hidden_size, self.experts
        n_out = E + self.identity
        logits = linear.linear(h, self.w_router, out_dtype=torch.float32)
        ids, weights = ops.moe_route(logits, self.correction, self.top, n_out, self.scores)
        rows, tile_expert = ops.moe_align(ids, E, ops.moe_tile_choice(ids.numel(), E, (W, self.expert_ff), h.dtype))
        if self.activation == "swiglu":
            gu = ops.grouped_gemm(h, self.w_up, rows, tile_expert, self.rt.empty(rows.numel(), 2 * self.expert_ff),
                                  gather_div=self.top)
            on_input = self.weight_on == "input"
            mid = ops.scaled_swiglu(gu, self.rt.empty(rows.numel(), self.expert_ff), weights.view(-1) if on_input else None, rows)
            if on_input:
                weights = None
        else:
            mid = ops.grouped_gemm(h, self.w_up, rows, tile_expert, self.rt.empty(rows.numel(), self.expert_ff),
                                   gather_div=self.top, act=self.activation)
        part = ops.grouped_gemm(mid, self.w_down, rows, tile_expert,
                                torch.empty((N * self.top, W), dtype=torch.float32, device=h.device), scatter=True)
        shared = gate = None
        if self.shared_ff:
            u = linear.linear(h, self.w_shared_up)
            shared = linear.linear(ops.gelu(u, torch.empty_like(u)), self.w_shared_down)
            gate = logits[:, n_out]
        out = torch.empty((N, W), dtype=torch.float32, device=h.device)
        return ops.moe_combine(part, ids, weights, h, E, out, shared, gate)


register_part("feed_forward", "routed_experts", RoutedExperts)
