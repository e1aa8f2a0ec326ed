"""Typed configuration of the Mifidra decoder.

config.json names the design in `architecture` and gives `vocab`, `width`, `norm.eps`, `logit_scale`, optionally
`loop` (`start`, `stop`, `times`: layers start .. stop - 1 run `times` times in a row) and `layers`, one entry a
layer: `type` ("parallel": softmax attention and the gated delta rule side by side), `mixer` (`left`, `right`,
`left_scale`, `right_scale`) and `mlp` (`{"kind": "dense", "ff"}`, `{"kind": "moe", "expert": {"ff"}, "router":
{"experts", "top", "groups": {"count", "keep"}}, "shared": {"ff"}}` or null).  Two sizes are in no key, the ranks of
the delta rule's two bottlenecks (its decay's and its gate's): the shapes of their tensors give them (`completed`);
`right.decay_rank` and `right.gate_rank` may state them, which a configuration without a file needs.  Every error
names its key.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, replace
from typing import Any, Dict, Mapping, Optional, Tuple

from .base import ConfigError, ModelConfig
from .vupelorn import Rotary, _get


@dataclass(frozen=True)
class SoftmaxSide:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[Rotary]

    @classmethod
    def from_dict(cls, d, where):
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: required key '{where}' is missing")
        heads = _get(d, "heads", where, least=1)
        dim = _get(d, "dim", where, least=1)
        rot = d.get("rot")
        c = cls(heads, _get(d, "kv_heads", where, least=1, default=heads), dim,
                _get(d, "vdim", where, least=1, default=dim), _get(d, "scale", where, float),
                None if rot is None else Rotary.from_dict(rot, where + ".rot", whole=dim - dim % 2))
        if c.heads % c.kv_heads:
            raise ConfigError(f"config.json: '{where}.heads' ({c.heads}) is no multiple of kv_heads ({c.kv_heads})")
        if c.rot is not None and c.rot.dims > c.dim:
            raise ConfigError(f"config.json: '{where}.rot.dims' ({c.rot.dims}) is more than dim ({c.dim})")
        return c

    def to_dict(self):
        d = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale, "vdim": self.vdim}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass(frozen=True)
class DeltaSide:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: Optional[int]  # None: the shape of the layer's first decay matrix says it
    gate_rank: Optional[int]  # None: the shape of the layer's first gate matrix says it

    @classmethod
    def from_dict(cls, d, where):
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: required key '{where}' is missing")
        heads = _get(d, "heads", where, least=1)
        dim = _get(d, "dim", where, least=1)
        c = cls(heads, _get(d, "kv_heads", where, least=1, default=heads), dim,
                _get(d, "vdim", where, least=1, default=dim), _get(d, "conv", where, least=1),
                _get(d, "decay_rank", where, least=1, default=None), _get(d, "gate_rank", where, least=1, default=None))
        if c.heads % c.kv_heads:
            raise ConfigError(f"config.json: '{where}.heads' ({c.heads}) is no multiple of kv_heads ({c.kv_heads})")
        return c

    def to_dict(self):
        d = {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}
        if self.decay_rank is not None:
            d["decay_rank"] = self.decay_rank
        if self.gate_rank is not None:
            d["gate_rank"] = self.gate_rank
        return d


@dataclass(frozen=True)
class FeedForward:
    kind: str  # "dense" | "moe"
    ff: int  # inner size (of an expert, for "moe")
    experts: int = 0
    top: int = 0
    groups: int = 0  # 0: the experts form no groups
    keep: int = 0
    shared_ff: int = 0  # 0: no shared expert

    @classmethod
    def from_dict(cls, d, where):
        kind = d.get("kind") if isinstance(d, dict) else None
        if kind == "dense":
            return cls("dense", _get(d, "ff", where, least=1))
        if kind != "moe":
            raise ConfigError(f"config.json: '{where}.kind' must be 'dense' or 'moe' (or mlp null), found {kind!r}")
        router, w = d.get("router"), where + ".router"
        groups = router.get("groups") if isinstance(router, dict) else None
        shared = d.get("shared")
        c = cls("moe", _get(d.get("expert"), "ff", where + ".expert", least=1), _get(router, "experts", w, least=1),
                _get(router, "top", w, least=1),
                0 if groups is None else _get(groups, "count", w + ".groups", least=1),
                0 if groups is None else _get(groups, "keep", w + ".groups", least=1),
                0 if shared is None else _get(shared, "ff", where + ".shared", least=1))
        if c.top > c.experts:
            raise ConfigError(f"config.json: '{w}.top' ({c.top}) is more than its {c.experts} experts")
        if c.groups:
            if c.experts % c.groups or c.keep > c.groups:
                raise ConfigError(f"config.json: '{w}.groups': {c.experts} experts do not form {c.groups} equal groups "
                                  f"of which {c.keep} are kept")
            if c.keep * (c.experts // c.groups) < c.top:
                raise ConfigError(f"config.json: '{w}.groups': {c.keep} groups of {c.experts // c.groups} experts "
                                  f"cannot give {c.top} experts")
        return c

    def to_dict(self):
        if self.kind == "dense":
            return {"ff": self.ff, "kind": "dense"}
        router: Dict[str, Any] = {"experts": self.experts, "top": self.top}
        if self.groups:
            router["groups"] = {"count": self.groups, "keep": self.keep}
        d: Dict[str, Any] = {"expert": {"ff": self.ff}, "kind": "moe", "router": router}
        if self.shared_ff:
            d["shared"] = {"ff": self.shared_ff}
        return d


@dataclass(frozen=True)
class MifidraLayer:
    type: str  # "parallel"
    left: SoftmaxSide
    right: DeltaSide
    left_scale: float
    right_scale: float
    mlp: Optional[FeedForward]

    @classmethod
    def from_dict(cls, d, i: int):
        where = f"layers[{i}]"
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: '{where}' must be an object")
        if d.get("type") != "parallel":
            raise ConfigError(f"config.json: '{where}.type' must be 'parallel', found {d.get('type')!r}")
        mixer = d.get("mixer")
        if not isinstance(mixer, dict):
            raise ConfigError(f"config.json: required key '{where}.mixer' is missing")
        w = where + ".mixer"
        mlp = d.get("mlp")
        return cls("parallel", SoftmaxSide.from_dict(mixer.get("left"), w + ".left"),
                   DeltaSide.from_dict(mixer.get("right"), w + ".right"), _get(mixer, "left_scale", w, float),
                   _get(mixer, "right_scale", w, float),
                   None if mlp is None else FeedForward.from_dict(mlp, where + ".mlp"))

    def to_dict(self):
        return {"mixer": {"left": self.left.to_dict(), "left_scale": self.left_scale, "right": self.right.to_dict(),
                          "right_scale": self.right_scale},
                "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass(frozen=True)
class Loop:
    start: int
    stop: int
    times: int

    def to_dict(self):
        return {"start": self.start, "stop": self.stop, "times": self.times}


@dataclass(frozen=True)
class MifidraConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    logit_scale: float
    loop: Optional[Loop]
    layers: Tuple[MifidraLayer, ...]
    architecture: str = "Mifidra"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MifidraConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        parsed = tuple(MifidraLayer.from_dict(x, i) for i, x in enumerate(layers))
        if not isinstance(d.get("norm"), dict):
            raise ConfigError("config.json: 'norm' must be an object")
        loop = None
        if d.get("loop") is not None:
            lp = d["loop"]
            loop = Loop(_get(lp, "start", "loop", least=0), _get(lp, "stop", "loop", least=0),
                        _get(lp, "times", "loop", least=1))
            if not loop.start <= loop.stop <= len(parsed):
                raise ConfigError(f"config.json: 'loop' runs layers {loop.start} to {loop.stop - 1} of {len(parsed)}")
        return cls(vocab=_get(d, "vocab", "config", least=1), width=_get(d, "width", "config", least=1),
                   norm_eps=_get(d["norm"], "eps", "norm", float),
                   logit_scale=_get(d, "logit_scale", "config", float, default=1.0), loop=loop, layers=parsed,
                   architecture=str(d.get("architecture", "Mifidra")))

    def run_order(self):
        """The layers in the order they run, as (layer, whether a pass after the first starts with it)."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        lp = self.loop
        order = [(i, False) for i in range(lp.start)]
        for t in range(lp.times):
            order += [(i, t > 0 and i == lp.start) for i in range(lp.start, lp.stop)]
        return order + [(i, False) for i in range(lp.stop, n)]

    def completed(self, shapes: Mapping[str, Tuple[int, ...]]) -> "MifidraConfig":
        """The sizes that no key gives, from the shapes of a file's tensors (name -> shape)."""
        layers = list(self.layers)
        for i, layer in enumerate(layers):
            right = layer.right
            for field, tensor in (("decay_rank", f"l{i}.mix.right.a1"), ("gate_rank", f"l{i}.mix.right.g1")):
                if getattr(right, field) is None:
                    shape = shapes.get(tensor)
                    if shape is None or len(shape) != 2:
                        raise ConfigError(f"layers[{i}]: the file has no matrix '{tensor}' to say the bottleneck's rank")
                    right = replace(right, **{field: int(shape[0])})
            layers[i] = replace(layer, right=right)
        return replace(self, layers=tuple(layers))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"architecture": self.architecture, "layers": [x.to_dict() for x in self.layers],
                             "logit_scale": self.logit_scale, "norm": {"eps": self.norm_eps}, "vocab": self.vocab,
                             "width": self.width}
        if self.loop is not None:
            d["loop"] = self.loop.to_dict()
        return copy.deepcopy(d)
