"""Typed configuration of the Kuvazen decoder and its translation into a ``ModelSpec``.

config.json: ``architecture`` "Kuvazen", ``vocab``, ``width``, ``norm.eps``, ``token_side.dim`` (absent or null: the
layers take no side input from the token), ``layers`` (one entry per layer: ``type``, the mixer: "mingru" {"width"} or
"attention" {"heads", "kv_heads", "dim", "vdim", "scale", "rot": {"base", "dims"}, "mask": {"size", "pool"}}; ``mlp``:
{"kind": "dense", "ff", "limit"}, {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}}, or null for a layer
without a feed-forward) and optionally ``loop`` {"start", "stop", "times"}: the layers start .. stop - 1 are walked
``times`` times in a row with the same weights, each walk with caches and states of its own.

Fixed by the design and therefore constants here: norms are layer norms with a weight and no bias (the embedding's rows
pass one too); every sublayer's result is multiplied by a stored vector before the sum; attention turns neighbouring
entries of q and k, turns its values over their whole size and the result back, and sees a window of tokens and pooled
blocks before it; the dense feed-forward clamps gate and up and uses sigmoid(1.702 g); routed experts are gated with
SiLU, scored by a sigmoid, and their weight scales what they read; tensors are named ``embed``, ``embed.norm``,
``side.embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.ls1``, ``l<i>.ls2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.side.*``,
``final.norm``, ``head``.
"""
from __future__ import annotations

import copy
import json
from dataclasses import dataclass
from typing import Optional, Tuple

from .gidurax import _need
from .registry import ConfigError, register_architecture
from .spec import ModelSpec, PartSpec, Run, layer

MIXERS = ("mingru", "attention")
GLU_ALPHA = 1.702      # the dense feed-forward's g * sigmoid(alpha g)


@dataclass(frozen=True)
class KuvazenConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[dict, ...]          # as config.json gives them (checked in __post_init__, never changed afterwards)
    side_dim: Optional[int] = None
    loop: Optional[Tuple[int, int, int]] = None     # (start, stop, times)

    architecture = "Kuvazen"

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
            if kind == "mingru":
                _need(m, "width", where + ".mixer")
            else:
                for k in ("heads", "kv_heads", "dim", "vdim"):
                    _need(m, k, where + ".mixer")
                _need(m, "scale", where + ".mixer", float)
                if m["heads"] % m["kv_heads"]:
                    raise ConfigError(f"config.json: {where}.mixer: {m['heads']} heads cannot share {m['kv_heads']} kv_heads")
                _need(m.get("rot"), "base", where + ".mixer.rot", float)
                _need(m.get("rot"), "dims", where + ".mixer.rot", positive=False)
                if m["rot"]["dims"] % 2 or m["rot"]["dims"] > m["dim"] or m["dim"] % 2 or m["vdim"] % 2:
                    raise ConfigError(f"config.json: {where}.mixer: entries turn in pairs: dim, vdim and rot.dims are even "
                                      f"and rot.dims is at most dim")
                _need(m.get("mask"), "size", where + ".mixer.mask")
                _need(m.get("mask"), "pool", where + ".mixer.mask")
            mlp = entry.get("mlp")
            if mlp is not None:
                if mlp.get("kind") == "dense":
                    _need(mlp, "ff", where + ".mlp")
                    _need(mlp, "limit", where + ".mlp", float)
                elif mlp.get("kind") == "moe":
                    _need(mlp.get("expert"), "ff", where + ".mlp.expert")
                    r = mlp.get("router")
                    _need(r, "experts", where + ".mlp.router")
                    _need(r, "top", where + ".mlp.router")
                    if r["top"] > r["experts"]:
                        raise ConfigError(f"config.json: {where}.mlp.router: top {r['top']} exceeds the experts there are")
                else:
                    raise ConfigError(f"config.json: {where}.mlp.kind is {mlp.get('kind')!r}; this design has 'dense' and 'moe'")
        if self.side_dim is not None and self.side_dim <= 0:
            raise ConfigError("token_side.dim must be positive")
        if self.loop is not None:
            start, stop, times = self.loop
            if not (0 <= start < stop <= len(self.layers)) or times <= 0:
                raise ConfigError(f"config.json: loop {{start: {start}, stop: {stop}, times: {times}}} does not name a "
                                  f"stretch of the {len(self.layers)} layers walked at least once")

    # ------------------------------------------------------------------ config.json
    @classmethod
    def from_dict(cls, d: dict) -> "KuvazenConfig":
        layers = d.get("layers")
        if not isinstance(layers, list):
            raise ConfigError("config.json lacks the list 'layers'")
        loop = d.get("loop")
        if loop is not None:
            loop = (_need(loop, "start", "loop", positive=False), _need(loop, "stop", "loop"), _need(loop, "times", "loop"))
        side = d.get("token_side")
        return cls(vocab=_need(d, "vocab", "config"), width=_need(d, "width", "config"),
                   norm_eps=_need(d.get("norm"), "eps", "norm", float),
                   layers=tuple(copy.deepcopy(e) for e in layers),
                   side_dim=_need(side, "dim", "token_side") if side is not None else None, loop=loop)

    def to_dict(self) -> dict:
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
             "layers": [copy.deepcopy(e) for e in self.layers]}
        if self.side_dim is not None:
            d["token_side"] = {"dim": self.side_dim}
        if self.loop is not None:
            d["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        return d

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
    def _mixer(self, i: int, entry: dict):
        """(mixer PartSpec, position PartSpec or None) of layer i."""
        m, p, W = entry["mixer"], f"l{i}.mix.", self.width
        if entry["type"] == "mingru":
            return PartSpec("mingru", p, {"hidden_size": W, "width": m["width"]}), None
        base, dims = float(m["rot"]["base"]), int(m["rot"]["dims"])
        position = PartSpec("rotary_pairs", p, {"width": m["dim"], "dims": dims, "theta": base})
        mixer = PartSpec("pooled_window_attention", p, {
            "hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"],
            "value_dim": m["vdim"], "scale": float(m["scale"]), "size": m["mask"]["size"], "pool": m["mask"]["pool"],
            "rotate_values": True, "value_theta": base})
        return mixer, position

    def _feed_forward(self, i: int, mlp: dict) -> PartSpec:
        p, W = f"l{i}.mlp.", self.width
        if mlp["kind"] == "dense":
            return PartSpec("clamped_glu", p, {"hidden_size": W, "intermediate_size": mlp["ff"], "limit": float(mlp["limit"]),
                                               "alpha": GLU_ALPHA})
        r = mlp["router"]
        return PartSpec("routed_experts", p, {
            "hidden_size": W, "expert_ff": mlp["expert"]["ff"], "experts": r["experts"], "identity": 0, "top": r["top"],
            "shared_ff": 0, "activation": "swiglu", "scores": "sigmoid", "correction": False, "weight_on": "input"})

    def order(self) -> Tuple[Run, ...]:
        n = len(self.layers)
        if self.loop is None:
            return tuple(Run(i) for i in range(n))
        start, stop, times = self.loop
        return tuple([Run(i) for i in range(start)] + [Run(i) for _ in range(times) for i in range(start, stop)] +
                     [Run(i) for i in range(stop, n)])

    def to_spec(self) -> ModelSpec:
        W, eps, n = self.width, self.norm_eps, len(self.layers)
        layers = []
        for i, entry in enumerate(self.layers):
            p = f"l{i}."
            mixer, position = self._mixer(i, entry)
            mlp = entry.get("mlp")

            def norm(name):
                return PartSpec("layer_norm", p, {"size": W, "eps": eps, "name": name})

            def scale(name):
                return PartSpec("layer_scale", p, {"size": W, "name": name})

            side = None if self.side_dim is None else PartSpec("token_side", p + "side.", {
                "hidden_size": W, "vocab_size": self.vocab, "dim": self.side_dim, "part": i, "parts": n, "eps": eps,
                "table_name": "side.embed"})
            layers.append(layer(
                "pre_norm_scaled_residual", position=position, mixer_norm=norm("norm1"), mixer=mixer, mixer_scale=scale("ls1"),
                feed_forward_norm=None if mlp is None else norm("norm2"),
                feed_forward=None if mlp is None else self._feed_forward(i, mlp),
                feed_forward_scale=None if mlp is None else scale("ls2"), token_input=side))
        return ModelSpec(
            architecture=self.architecture, hidden_size=W, vocab_size=self.vocab,
            embedding=PartSpec("token_embedding", "", {
                "vocab_size": self.vocab, "hidden_size": W, "name": "embed",
                "norm": PartSpec("layer_norm", "embed.", {"size": W, "eps": eps, "name": "norm"})}),
            layers=tuple(layers), order=self.order(),
            final_norm=PartSpec("layer_norm", "final.", {"size": W, "eps": eps, "name": "norm"}),
            head=PartSpec("lm_head", "", {"hidden_size": W, "vocab_size": self.vocab, "tied_to": None, "name": "head"}),
            ignorable=tuple(f"l{i}.{t}" for i, e in enumerate(self.layers) if e.get("mlp") is None for t in ("norm2", "ls2")),
        )


register_architecture(KuvazenConfig.architecture, KuvazenConfig, model_type="kuvazen")
