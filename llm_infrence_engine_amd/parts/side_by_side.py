"""Two mixers side by side: both read the same input h, and the layer's mixer result is a sum of the two.

``combine`` = "scaled": left_scale * left(h) + right_scale * right(h).  With both scales one (a configuration may hand the
scales to the halves themselves, where they ride on a kernel that is there anyway) every half adds its result into the
residual stream through its own last product, and only what a half hands back is summed here.
``combine`` = "normed_mean": (RMS(left(h)) o w_left + RMS(right(h)) o w_right) / 2, each result divided by its root mean
square over the model's width (eps inside the root) and multiplied by a stored weight of its own (``left_norm_name`` /
``right_norm_name`` after the prefix).

``left`` and ``right`` are ``PartSpec``s of mixers of any kind (``left_position`` / ``right_position``: their position
encodings).  At most one of the two keeps a cache of keys; their fixed-size states lie side by side in the run's state
tensors, the left one's first.  The sum is float and goes straight into the float residual stream."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import TensorSpec
from .base import Mixer, StateView, build_part, register_part, weakest


def _as_list(need):
    return [] if need is None else (list(need) if isinstance(need, (tuple, list)) else [need])


class SideBySide(Mixer):
    COMBINE = ("scaled", "normed_mean")

    def __init__(self, prefix: str, position, hidden_size: int, left, right, combine: str = "scaled", left_scale: float = 1.0,
                 right_scale: float = 1.0, eps: float = 0.0, left_position=None, right_position=None,
                 left_norm_name: str = "left.out", right_norm_name: str = "right.out"):
        if combine not in self.COMBINE:
            raise ValueError(f"no way {combine!r} of joining two mixers; there are {', '.join(self.COMBINE)}")
        self.prefix, self.hidden_size, self.combine, self.eps = prefix, hidden_size, combine, float(eps)
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self.left_norm_name, self.right_norm_name = left_norm_name, right_norm_name
        self.halves = []
        for spec, pos in ((left, left_position), (right, right_position)):
            built_pos = build_part("position", pos) if pos is not None else None
            self.halves.append(build_part("mixer", spec, position=built_pos))
        if sum(m.cache_need() is not None for m in self.halves) > 1:
            raise ValueError("of two mixers side by side at most one may keep a cache of keys")
        self.norm_left = self.norm_right = None

    @property
    def graph_safe(self):
        return weakest(m.graph_safe for m in self.halves)

    # ---- weights
    def tensor_specs(self):
        specs = [s for m in self.halves for s in m.tensor_specs()]
        if self.combine == "normed_mean":
            specs += [TensorSpec(self.prefix + self.left_norm_name, (self.hidden_size,), "norm"),
                      TensorSpec(self.prefix + self.right_norm_name, (self.hidden_size,), "norm")]
        return specs

    def load(self, get, rt):
        self.rt = rt
        for m in self.halves:
            m.load(get, rt)
        if self.combine == "normed_mean":
            self.norm_left, self.norm_right = (get(s) for s in SideBySide.tensor_specs(self)[-2:])

    # ---- cache and state
    def cache_need(self):
        for m in self.halves:
            need = m.cache_need()
            if need is not None:
                return need
        return None

    def state_need(self):
        needs = [n for m in self.halves for n in _as_list(m.state_need())]
        if not needs:
            return None
        return needs[0] if len(needs) == 1 else tuple(needs)

    def _state_of(self, which: int, state):
        """The half's own share of the state tensors, shaped as the half declared it."""
        if state is None:
            return None
        counts = [len(_as_list(m.state_need())) for m in self.halves]
        if counts[which] == 0:
            return None
        slots = state.slots if isinstance(state.slots, (tuple, list)) else (state.slots,)
        at = sum(counts[:which])
        mine = tuple(slots[at:at + counts[which]])
        declared = self.halves[which].state_need()
        return StateView(mine if isinstance(declared, (tuple, list)) else mine[0])

    # ---- step
    def forward(self, h, ctx, kv, state):
        x = torch.empty((ctx.num_tokens, self.hidden_size), dtype=torch.float32, device=h.device).zero_()
        self.forward_residual(h, ctx, kv, state, x)
        return x

    def forward_residual(self, h, ctx, kv, state, x):
        if self.combine == "scaled" and self.left_scale == 1.0 and self.right_scale == 1.0:
            handed = []
            for i, m in enumerate(self.halves):
                mine = kv if m.cache_need() is not None else None
                r = m.forward_residual(h, ctx, mine, self._state_of(i, state), x)
                if r is not None:
                    handed.append(r)
            if len(handed) == 2:
                ops.pair_sum(x, handed[0], handed[1])
            elif handed:
                ops.residual_add(x, handed[0])
            return None
        results = []
        for i, m in enumerate(self.halves):
            mine = kv if m.cache_need() is not None else None
            results.append(m.forward(h, ctx, mine, self._state_of(i, state)))
        a, b = results
        if self.combine == "scaled":
            ops.pair_sum(x, a, b, self.left_scale, self.right_scale)
        else:
            ops.pair_sum(x, a, b, 0.5, 0.5, self.norm_left, self.norm_right, self.eps)
        return None


register_part("mixer", "side_by_side", SideBySide)
