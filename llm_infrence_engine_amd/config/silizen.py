"""Typed configuration of the Silizen decoder and its translation into a ``ModelSpec``.

config.json: ``architecture`` "Silizen", ``vocab``, ``width``, ``norm.eps``, ``logit_scale``, ``layers`` (one entry per layer:
``type`` "parallel", "parallel_2" or "wkv"; ``mixer``, its sizes and constants; ``mlp``: {"kind": "dense", "ff"} or null for
a layer without a feed-forward) and optionally ``loop`` {"start", "stop", "times"}: the layers start .. stop - 1 are walked
``times`` times in a row with the same weights, each walk with caches and states of its own.

"parallel":   {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "softcap", "rot": {"base", "dims", "scaling": {"factor",
              "low", "high", "original"} or absent}}, "right": {"heads", "dim", "vdim", "tau"}, "left_scale", "right_scale"}
"parallel_2": {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "mask": {"size"}}, "right": {"heads", "kv_heads", "dim",
              "vdim", "conv"}}
"wkv":        {"heads", "dim"}
The ranks of the low-rank maps (the decays' and the delta rule's gate) are the shapes of their tensors (``with_tensor_shapes``),
or stated as ``decay_rank`` / ``gate_rank`` in the mixer's entry.

Fixed by the design and therefore constants here: a layer has one layer norm (weight and bias) that its mixer and its
feed-forward both read, and adds their sum to the residual stream; "parallel" and "parallel_2" run attention (left) beside a
recurrence (right) on the same input; both attentions add one to the softmax's denominator and gate every head's result by
a sigmoid; the first normalises its heads with weights and rotates half-split pairs, the second normalises them without
weights and takes 2^(-8 (h + 1) / H) (i - j) off the scores inside a sliding window; feed-forwards are gated with the tanh
gelu; before every walk over the looped stretch the residual stream and the embedding's output pass ``loop.in`` together; the
head is the embedding table, and the logits are scaled; tensors are named ``embed``, ``loop.in``, ``l<i>.norm1``,
``l<i>.norm1.b``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``final.norm.b``.
"""
from __future__ import annotations

import copy
import json
from dataclasses import dataclass, replace
from typing import Optional, Tuple

from .gidurax import _need
from .registry import ConfigError, register_architecture
from .spec import ModelSpec, PartSpec, Run, layer

MIXERS = ("parallel", "parallel_2", "wkv")
SLOPE_BASE = 8.0       # the distance penalty of head h of H: 2^(-8 (h + 1) / H) per token of distance


def _rank_names(i: int, entry: dict):
    """{key in the mixer's entry (dotted): the tensor whose first dimension is that rank} of layer i."""
    p = f"l{i}.mix."
    if entry["type"] == "parallel":
        return {"right.decay_rank": p + "right.a1"}
    if entry["type"] == "parallel_2":
        return {"right.decay_rank": p + "right.a1", "right.gate_rank": p + "right.g1"}
    return {"decay_rank": p + "w1"}


def _get(m: dict, dotted: str):
    for k in dotted.split("."):
        m = m.get(k) if isinstance(m, dict) else None
    return m


@dataclass(frozen=True)
class SilizenConfig:
    vocab: int
    width: int
    norm_eps: float
    logit_scale: float
    layers: Tuple[dict, ...]          # as config.json gives them (checked in __post_init__, never changed afterwards)
    loop: Optional[Tuple[int, int, int]] = None     # (start, stop, times)

    architecture = "Silizen"

    def __hash__(self):
        return hash(json.dumps(self.to_dict(), sort_keys=True))

    def __post_init__(self):
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.norm_eps >= 0:
            raise ConfigError(f"norm.eps must be >= 0, got {self.norm_eps}")
        if not self.layers:
            raise ConfigError("config.json: 'layers' is empty")
        for i, entry in enumerate(self.layers):
            where = f"layers[{i}]"
            kind = entry.get("type") if isinstance(entry, dict) else None
            if kind not in MIXERS:
                raise ConfigError(f"config.json: {where}.type is {kind!r}; this design has {', '.join(MIXERS)}")
            m = entry.get("mixer")
            if kind == "wkv":
                for k in ("heads", "dim"):
                    _need(m, k, where + ".mixer")
            else:
                left, right = (m or {}).get("left"), (m or {}).get("right")
                for k in ("heads", "kv_heads", "dim", "vdim"):
                    _need(left, k, where + ".mixer.left")
                _need(left, "scale", where + ".mixer.left", float)
                if left["heads"] % left["kv_heads"]:
                    raise ConfigError(f"config.json: {where}.mixer.left: {left['heads']} heads cannot share {left['kv_heads']} kv_heads")
                if kind == "parallel":
                    if left.get("softcap") is not None and not _need(left, "softcap", where + ".mixer.left", float) > 0:
                        raise ConfigError(f"config.json: {where}.mixer.left.softcap must be positive")
                    rot = left.get("rot")
                    if rot is not None:
                        _need(rot, "base", where + ".mixer.left.rot", float)
                        dims = _need(rot, "dims", where + ".mixer.left.rot", positive=False)
                        if dims % 2 or dims > left["dim"]:
                            raise ConfigError(f"config.json: {where}.mixer.left.rot.dims must be even and at most dim")
                        if rot.get("scaling") is not None:
                            for k in ("factor", "low", "high", "original"):
                                _need(rot["scaling"], k, where + ".mixer.left.rot.scaling", float)
                    for k in ("heads", "dim", "vdim"):
                        _need(right, k, where + ".mixer.right")
                    if not _need(right, "tau", where + ".mixer.right", float) > 0:
                        raise ConfigError(f"config.json: {where}.mixer.right.tau must be positive")
                    _need(m, "left_scale", where + ".mixer", float)
                    _need(m, "right_scale", where + ".mixer", float)
                else:
                    if left.get("mask") is not None:
                        _need(left["mask"], "size", where + ".mixer.left.mask")
                    for k in ("heads", "kv_heads", "dim", "vdim", "conv"):
                        _need(right, k, where + ".mixer.right")
                    if right["heads"] % right["kv_heads"]:
                        raise ConfigError(f"config.json: {where}.mixer.right: {right['heads']} heads cannot share "
                                          f"{right['kv_heads']} kv_heads")
            mlp = entry.get("mlp")
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp.kind is {mlp.get('kind')!r}; this design has 'dense'")
                _need(mlp, "ff", where + ".mlp")
        if self.loop is not None:
            start, stop, times = self.loop
            if not (0 <= start < stop <= len(self.layers)) or times <= 0:
                raise ConfigError(f"config.json: loop {{start: {start}, stop: {stop}, times: {times}}} does not name a "
                                  f"stretch of the {len(self.layers)} layers walked at least once")

    # ------------------------------------------------------------------ config.json
    @classmethod
    def from_dict(cls, d: dict) -> "SilizenConfig":
        layers = d.get("layers")
        if not isinstance(layers, list):
            raise ConfigError("config.json lacks the list 'layers'")
        loop = d.get("loop")
        if loop is not None:
            loop = (_need(loop, "start", "loop", positive=False), _need(loop, "stop", "loop"), _need(loop, "times", "loop"))
        return cls(vocab=_need(d, "vocab", "config"), width=_need(d, "width", "config"),
                   norm_eps=_need(d.get("norm"), "eps", "norm", float),
                   logit_scale=_need(d, "logit_scale", "config", float) if d.get("logit_scale") is not None else 1.0,
                   layers=tuple(copy.deepcopy(e) for e in layers), loop=loop)

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
             "logit_scale": self.logit_scale, "layers": [copy.deepcopy(e) for e in self.layers]}
        if self.loop is not None:
            d["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        return d

    def with_tensor_shapes(self, shape_of) -> "SilizenConfig":
        """The ranks that config.json leaves to the tensors: ``shape_of(name)`` gives a tensor's shape or None."""
        layers = []
        for i, entry in enumerate(self.layers):
            entry = copy.deepcopy(entry)
            for dotted, tensor in _rank_names(i, entry).items():
                if _get(entry["mixer"], dotted) is None:
                    shape = shape_of(tensor)
                    if shape is not None:
                        *path, key = dotted.split(".")
                        m = entry["mixer"]
                        for k in path:
                            m = m[k]
                        m[key] = int(shape[0])
            layers.append(entry)
        return replace(self, layers=tuple(layers))

    def _rank(self, i: int, entry: dict, dotted: str) -> int:
        r = _get(entry["mixer"], dotted)
        if r is None:
            raise ConfigError(f"config.json: layers[{i}].mixer.{dotted} is not stated and no checkpoint gave the shape of "
                              f"{_rank_names(i, entry)[dotted]}")
        return int(r)

    # ------------------------------------------------------------------ derived sizes
    @property
    def num_params(self) -> int:
        from ..parts.model import Model

        total = 0
        for s in Model(self.to_spec()).tensor_specs():
            n = 1
            for d in s.shape:
                n *= d
            total += n
        return total

    # ------------------------------------------------------------------ the model as data
    def _attention(self, p: str, left: dict, kind: str, out_scale: float = 1.0) -> Tuple[PartSpec, PartSpec]:
        """(mixer PartSpec, position PartSpec) of an attention half; ``out_scale``: the half's weight in the mixer's sum."""
        W, eps = self.width, self.norm_eps
        names = {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g"}
        common = {"hidden_size": W, "num_heads": left["heads"], "num_kv_heads": left["kv_heads"], "head_dim": left["dim"],
                  "value_dim": left["vdim"], "scale": float(left["scale"]), "out_bias": False, "sink": "zero", "gate": True,
                  "names": names, "bias_suffix": ".b", "out_scale": float(out_scale)}
        if kind == "parallel":
            rot = left.get("rot") or {}
            position = PartSpec("qk_norm_rotary_half", p, {
                "head_dim": left["dim"], "eps": eps, "weighted": True, "dims": int(rot.get("dims", 0)),
                "base": float(rot.get("base", 10000.0)),
                "scaling": tuple(sorted(rot["scaling"].items())) if rot.get("scaling") is not None else None})
            softcap = left.get("softcap")
            return PartSpec("gqa_attention", p, dict(common, qkv_bias=False, softcap=None if softcap is None else float(softcap))), position
        position = PartSpec("qk_norm_rotary_half", p, {"head_dim": left["dim"], "eps": eps, "weighted": False, "dims": 0})
        window = left["mask"]["size"] if left.get("mask") is not None else None
        return PartSpec("gqa_attention", p, dict(common, qkv_bias=True, window=window, slope_base=SLOPE_BASE)), position

    def _mixer(self, i: int, entry: dict) -> PartSpec:
        m, p, W, eps = entry["mixer"], f"l{i}.mix.", self.width, self.norm_eps
        kind = entry["type"]
        if kind == "wkv":
            return PartSpec("wkv", p, {"hidden_size": W, "heads": m["heads"], "dim": m["dim"], "eps": eps,
                                       "decay_rank": self._rank(i, entry, "decay_rank")})
        r = m["right"]
        if kind == "parallel":
            # the halves' weights ride on kernels that are there anyway (the attention's normalisation, the read-out's norm),
            # so that each half's output product can add straight into the residual stream
            left, left_position = self._attention(p + "left.", m["left"], kind, out_scale=float(m["left_scale"]))
            right = PartSpec("gated_linear_attention", p + "right.", {
                "hidden_size": W, "heads": r["heads"], "dim": r["dim"], "vdim": r["vdim"], "tau": float(r["tau"]), "eps": eps,
                "decay_rank": self._rank(i, entry, "right.decay_rank"), "out_scale": float(m["right_scale"])})
            return PartSpec("side_by_side", p, {"hidden_size": W, "left": left, "right": right, "left_position": left_position,
                                                "combine": "scaled"})
        left, left_position = self._attention(p + "left.", m["left"], kind)
        right = PartSpec("gated_delta", p + "right.", {
            "hidden_size": W, "heads": r["heads"], "kv_heads": r["kv_heads"], "dim": r["dim"], "vdim": r["vdim"],
            "taps": r["conv"], "eps": eps, "decay": "channel", "gate": "low_rank_sigmoid",
            "decay_rank": self._rank(i, entry, "right.decay_rank"), "gate_rank": self._rank(i, entry, "right.gate_rank")})
        return PartSpec("side_by_side", p, {"hidden_size": W, "left": left, "right": right, "left_position": left_position,
                                            "combine": "normed_mean", "eps": eps})

    def order(self) -> Tuple[Run, ...]:
        n = len(self.layers)
        if self.loop is None:
            return tuple(Run(i) for i in range(n))
        start, stop, times = self.loop
        runs = [Run(i) for i in range(start)]
        for t in range(times):
            runs += [Run(i, opens_pass=t if i == start else None) for i in range(start, stop)]
        return tuple(runs + [Run(i) for i in range(stop, n)])

    def to_spec(self) -> ModelSpec:
        W, eps = self.width, self.norm_eps
        layers = []
        for i, entry in enumerate(self.layers):
            p = f"l{i}."
            mlp = entry.get("mlp")
            layers.append(layer(
                "parallel_residual",
                mixer_norm=PartSpec("layer_norm", p, {"size": W, "eps": eps, "name": "norm1", "bias_name": "norm1.b"}),
                mixer=self._mixer(i, entry),
                feed_forward=None if mlp is None else PartSpec("gated_glu", p + "mlp.", {
                    "hidden_size": W, "intermediate_size": mlp["ff"], "activation": "gelu_tanh"})))
        return ModelSpec(
            architecture=self.architecture, hidden_size=W, vocab_size=self.vocab,
            embedding=PartSpec("token_embedding", "", {"vocab_size": self.vocab, "hidden_size": W, "name": "embed"}),
            layers=tuple(layers), order=self.order(),
            final_norm=PartSpec("layer_norm", "final.", {"size": W, "eps": eps, "name": "norm", "bias_name": "norm.b",
                                                         "gain": self.logit_scale}),
            head=PartSpec("lm_head", "", {"hidden_size": W, "vocab_size": self.vocab, "tied_to": "embed", "name": "head"}),
            pass_entry=PartSpec("pass_mix", "loop.", {"hidden_size": W, "name": "in"}) if self.loop is not None else None,
        )


register_architecture(SilizenConfig.architecture, SilizenConfig, model_type="silizen")
