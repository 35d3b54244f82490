"""Arrangements of a layer's parts.

``pre_norm_residual``: x = x + mixer(norm(x)); x = x + feed_forward(norm(x)) (src/miniserve/model.py:184-185).
The residual stream x is float.  A part either adds its result into x itself (its last matrix product does
it as an epilogue) or hands the addend on, and the sum is fused into the norm that follows; a block hands its
own last addend on as ``pending``."""
from __future__ import annotations

from ..kernels import ops
from .base import Block, register_part


class PreNormResidual(Block):
    takes = {"position": "position", "mixer_norm": "norm", "mixer": "mixer", "feed_forward_norm": "norm",
             "feed_forward": "feed_forward"}
    optional = ("position",)

    def forward(self, x, pending, ctx, kv, state):
        norm = self.mixer_norm.lazy if self.mixer.accepts_lazy_norm else self.mixer_norm.forward
        a = self.mixer.forward_residual(norm(x, delta=pending), ctx, kv, state, x)
        norm = self.feed_forward_norm.lazy if self.feed_forward.accepts_lazy_norm else self.feed_forward_norm.forward
        return self.feed_forward.forward_residual(norm(x, delta=a), ctx, x)


class ParallelResidual(Block):
    """x <- x + mixer(f(norm1(x))) + feed_forward(norm2(x)): both branches read the same x.  ``input_filter``
    (optional) is a map over time laid before the mixer's input, f; without a feed-forward the layer is
    x <- x + mixer(f(norm1(x))).  A layer with a feed-forward and no ``feed_forward_norm`` has one norm that both
    branches read: x <- x + mixer(f(h)) + feed_forward(h), h = norm1(x)."""

    takes = {"position": "position", "mixer_norm": "norm", "input_filter": "filter", "mixer": "mixer",
             "feed_forward_norm": "norm", "feed_forward": "feed_forward"}
    optional = ("position", "input_filter", "feed_forward_norm", "feed_forward")

    def forward(self, x, pending, ctx, kv, state):
        # x holds the sum both branches read before either adds to it; the two norms share their pass over x
        if self.feed_forward is not None and self.feed_forward_norm is None:
            h = h2 = self.mixer_norm.forward(x, delta=pending)
        elif self.feed_forward is not None and hasattr(self.mixer_norm, "forward_pair"):
            h, h2 = self.mixer_norm.forward_pair(self.feed_forward_norm, x, delta=pending)
        else:
            h = self.mixer_norm.forward(x, delta=pending)
            h2 = self.feed_forward_norm.forward(x) if self.feed_forward is not None else None
        if self.input_filter is not None:
            h = self.input_filter.forward(h, ctx, self.state_of("input_filter", state))
        a = self.mixer.forward_residual(h, ctx, kv, self.state_of("mixer", state), x)
        if self.feed_forward is None:
            return a
        b = self.feed_forward.forward_residual(h2, ctx, x)
        if a is not None and b is not None:
            ops.residual_add(x, a)
            return b
        return a if b is None else b


class SandwichResidual(Block):
    """x <- x + post1(mixer(norm1(x)));  x <- x + post2(feed_forward(norm2(x))): every sublayer is normalised before it
    and after it; the second norm's weight carries whatever constant the sublayer is weighted with in the sum
    (``rms_norm(gain=...)``).  The sum into x and the norm that the next sublayer of the layer reads are one pass.
    Without a feed-forward the layer is its first line."""

    takes = {"position": "position", "mixer_norm": "norm", "mixer": "mixer", "mixer_post_norm": "norm",
             "feed_forward_norm": "norm", "feed_forward": "feed_forward", "feed_forward_post_norm": "norm"}
    optional = ("position", "feed_forward_norm", "feed_forward", "feed_forward_post_norm")

    def forward(self, x, pending, ctx, kv, state):
        h = self.mixer_norm.forward(x, delta=pending)
        y = self.mixer.forward(h, ctx, kv, state)
        if self.feed_forward is None:
            self.mixer_post_norm.add_normed(x, y)
            return None
        h = self.mixer_post_norm.add_normed(x, y, then=self.feed_forward_norm)
        self.feed_forward_post_norm.add_normed(x, self.feed_forward.forward(h, ctx))
        return None


class ScaledPreNormResidual(Block):
    """x <- x + s1 o mixer(norm1(x));  x <- x + s2 o feed_forward(norm2(x));  then, if the layer has one, the token's own
    input (``token_input``) into x.  s1, s2 (``mixer_scale``, ``feed_forward_scale``; optional) are stored vectors.  Every
    scaled sum rides on the kernel that reads x next: the second norm, the token input, or a sum of its own.  Without a
    feed-forward the layer is its first line (and the token input)."""

    takes = {"position": "position", "mixer_norm": "norm", "mixer": "mixer", "mixer_scale": "scale",
             "feed_forward_norm": "norm", "feed_forward": "feed_forward", "feed_forward_scale": "scale",
             "token_input": "token_input"}
    optional = ("position", "mixer_scale", "feed_forward_norm", "feed_forward", "feed_forward_scale", "token_input")

    @staticmethod
    def _normed(norm, x, delta, scale):
        if delta is not None and scale is not None and not getattr(norm, "takes_delta_scale", False):
            ops.layer_norm(x, None, 0.0, None, delta=delta, delta_scale=scale)      # the scaled sum alone
            return norm.forward(x)
        return norm.forward(x, delta=delta, delta_scale=scale) if scale is not None else norm.forward(x, delta=delta)

    def forward(self, x, pending, ctx, kv, state):
        y = self.mixer.forward(self.mixer_norm.forward(x, delta=pending), ctx, kv, state)
        scale = self.mixer_scale.vector if self.mixer_scale is not None else None
        if self.feed_forward is not None:
            y = self.feed_forward.forward(self._normed(self.feed_forward_norm, x, y, scale), ctx)
            scale = self.feed_forward_scale.vector if self.feed_forward_scale is not None else None
        if self.token_input is not None:
            self.token_input.forward(x, ctx, delta=y, delta_scale=scale)
        else:
            ops.layer_norm(x, None, 0.0, None, delta=y, delta_scale=scale)
        return None


register_part("block", "pre_norm_residual", PreNormResidual)
register_part("block", "pre_norm_scaled_residual", ScaledPreNormResidual)
register_part("block", "sandwich_residual", SandwichResidual)
register_part("block", "parallel_residual", ParallelResidual)
