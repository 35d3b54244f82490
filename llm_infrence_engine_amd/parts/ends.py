"""The model's two ends: token embedding (a row gather into the float residual stream,
src/miniserve/model.py:229) and the output head (a matrix product with the head's own matrix or, when
tied, the embedding table, model.py:204-206, 237).  Logits are float."""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import Embedding, Head, PassEntry, build_part, register_part


class TokenEmbedding(Embedding):
    def __init__(self, prefix: str, vocab_size: int, hidden_size: int, name: str = "weight", scale: float = 1.0, norm=None):
        """``scale``: every row is multiplied by it on its way into the float residual stream.  ``norm``: the
        ``PartSpec`` of a norm that the rows pass right after (one with ``normalize_``), or None."""
        self.prefix, self.vocab_size, self.hidden_size, self.name = prefix, vocab_size, hidden_size, name
        self.scale = float(scale)
        self.norm = build_part("norm", norm) if norm is not None else None
        if self.norm is not None and not hasattr(self.norm, "normalize_"):
            raise ValueError(f"the norm {norm.kind!r} cannot be applied in place to the embedding's rows")

    def tensor_specs(self):
        return [TensorSpec(self.prefix + self.name, (self.vocab_size, self.hidden_size))] + \
            (self.norm.tensor_specs() if self.norm is not None else [])

    def load(self, get, rt):
        self.rt = rt
        self.weight = get(TokenEmbedding.tensor_specs(self)[0])
        if self.norm is not None:
            self.norm.load(get, rt)

    def forward(self, ctx):
        out = self.rt.empty(ctx.num_tokens, self.hidden_size, dtype=torch.float32)
        ops.embed(ctx.token_ids, self.weight, out, self.scale)
        return self.norm.normalize_(out) if self.norm is not None else out


class LMHead(Head):
    accepts_lazy_norm = True

    def __init__(self, prefix: str, hidden_size: int, vocab_size: int, tied_to=None, name: str = "weight"):
        self.prefix, self.hidden_size, self.vocab_size, self.tied_to, self.name = prefix, hidden_size, vocab_size, tied_to, name

    def tensor_specs(self):
        name = self.tied_to or self.prefix + self.name
        return [TensorSpec(name, (self.vocab_size, self.hidden_size))]

    def ignorable(self):
        """A tied head ignores a copy of its own that the checkpoint may still carry."""
        return [self.prefix + self.name] if self.tied_to else []

    def load(self, get, rt):
        self.rt = rt
        self.weight = linear.prepare_weight(get(self.tensor_specs()[0]))

    def forward(self, h):
        return linear.linear(h, self.weight, out_dtype=torch.float32)


class PassStep(PassEntry):
    """Before pass t: x <- x + e (for t > 0, with ``readd_embedding``; e is x as the embedding left it) + step[t], where
    ``step`` is a stored table [times, hidden_size] (tensor ``name``) with one row per pass."""

    def __init__(self, prefix: str, hidden_size: int, times: int, name: str = "step", readd_embedding: bool = True):
        if times <= 0:
            raise ValueError("a stretch of layers is walked at least once")
        self.prefix, self.hidden_size, self.times, self.name = prefix, hidden_size, times, name
        self.keeps_embedding = bool(readd_embedding) and times > 1

    def tensor_specs(self):
        return [TensorSpec(self.prefix + self.name, (self.times, self.hidden_size), "bias")]

    def load(self, get, rt):
        self.rt = rt
        self.step = get(self.tensor_specs()[0])

    def forward(self, x, kept, t):
        if not 0 <= t < self.times:
            raise ValueError(f"pass {t} of {self.times}")
        ops.add_rows(x, kept if (t > 0 and self.keeps_embedding) else None, self.step[t])


class PassMix(PassEntry):
    """Before every pass (the first too): x <- M [x ; e], with e the residual stream as the embedding left it and M a
    stored matrix [hidden_size, 2 hidden_size] (tensor ``name``) whose first half of columns meets x.  The product reads
    x and e rounded to the matrices' type and leaves as float, the new residual stream."""

    keeps_embedding = True

    def __init__(self, prefix: str, hidden_size: int, name: str = "in"):
        self.prefix, self.hidden_size, self.name = prefix, hidden_size, name

    def tensor_specs(self):
        return [TensorSpec(self.prefix + self.name, (self.hidden_size, 2 * self.hidden_size))]

    def load(self, get, rt):
        self.rt = rt
        self.weight = linear.prepare_weight(get(self.tensor_specs()[0]))

    def forward(self, x, kept, t):
        both = ops.concat_rows(x, kept, self.rt.empty(x.shape[0], 2 * self.hidden_size))
        return linear.linear(both, self.weight, out_dtype=torch.float32)


register_part("pass_entry", "pass_step", PassStep)
register_part("pass_entry", "pass_mix", PassMix)
register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "lm_head", LMHead)
