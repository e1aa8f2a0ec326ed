"""Typed configuration of the Sofinex decoder.

config.json names the design in `architecture` and gives `vocab`, `width`, `norm.eps`, `embedding.scale`,
optionally `loop` (`start`, `stop`, `times`: layers start .. stop - 1 run `times` times in a row) and `layers`, one
entry a layer: `type`, `mixer` and `mlp`.

* type "attention": differential attention.  `mixer`: `heads`, `kv_heads`, `dim` (of one map's queries and keys),
  `vdim`, `scale`, `diff`, `mask.size` (the sliding window; no `mask`: every earlier position) and `rot` (`base`,
  `dims`, `scaling`).
* type "parallel": `mixer.left` is windowed softmax attention with a learned sink (the same keys but `diff`),
  `mixer.right` the gated delta rule (`heads`, `kv_heads`, `dim`, `vdim`, `conv`).
* `rot.scaling` with `low` and `high` (and `factor`, `original`) blends the frequencies by wavelength; with `fast` and
  `slow` it ramps over the pairs and stretches cos and sin (YaRN).
* `mlp`: `{"kind": "dense", "ff"}`, `{"kind": "moe", "expert": {"ff"}, "router": {"experts", "top", "identity",
  "groups": {"count", "keep"}}, "shared": {"ff"}}` or null.

Two sizes are in no key, the ranks of the delta rule's two bottlenecks: the shapes of their tensors give them
(`completed`); `right.decay_rank` and `right.gate_rank` may state them, which a configuration without a file needs.
Every error names its key.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, replace
from typing import Any, Dict, Mapping, Optional, Tuple

from .base import ConfigError, ModelConfig
from .mifidra import DeltaSide, Loop
from .vupelorn import _get


@dataclass(frozen=True)
class RotaryTurn:
    base: float
    dims: int
    scaling: Optional[Tuple[Tuple[str, float], ...]]  # the scaling's keys and numbers, sorted by key

    @classmethod
    def from_dict(cls, d, where, whole: int):
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: '{where}' must be an object")
        sc, scaling = d.get("scaling"), None
        if sc is not None:
            w = where + ".scaling"
            keys = ("factor", "original", "low", "high") if isinstance(sc, dict) and "low" in sc \
                else ("factor", "original", "fast", "slow")
            vals = {k: _get(sc, k, w, float) for k in keys}
            if any(not v > 0 for v in vals.values()) or vals.get("low") == vals.get("high", 0.0):
                raise ConfigError(f"config.json: '{w}' needs positive numbers ({', '.join(keys)}; low and high differ)")
            scaling = tuple(sorted(vals.items()))
        c = cls(_get(d, "base", where, float), _get(d, "dims", where, least=2, default=whole - whole % 2), scaling)
        if c.dims % 2 or c.dims > whole or not c.base > 0:
            raise ConfigError(f"config.json: '{where}.dims' must be even and at most {whole}, '{where}.base' positive")
        return c

    def to_dict(self):
        d: Dict[str, Any] = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            d["scaling"] = dict(self.scaling)
        return d

    def as_parameters(self) -> Dict[str, Any]:
        """What the attention parts take as `rotary` (pairs (i, i + dims / 2))."""
        scaling = None
        if self.scaling is not None:
            sc = dict(self.scaling)
            if "low" in sc:
                scaling = {"rope_type": "llama3", "factor": sc["factor"], "low_freq_factor": sc["low"],
                           "high_freq_factor": sc["high"], "original_max_position_embeddings": sc["original"]}
            else:
                scaling = {"rope_type": "yarn", "factor": sc["factor"], "original": sc["original"], "fast": sc["fast"],
                           "slow": sc["slow"]}
        return {"dims": self.dims, "base": self.base, "scaling": scaling, "pairing": "half"}


@dataclass(frozen=True)
class WindowedHeads:
    """Softmax attention's sizes; `diff` is None for the plain kind and the constant of differential attention."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int  # 0: every earlier position
    rot: Optional[RotaryTurn]
    diff: Optional[float] = None

    @classmethod
    def from_dict(cls, d, where, differential: bool):
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: required key '{where}' is missing")
        heads = _get(d, "heads", where, least=1)
        dim = _get(d, "dim", where, least=1)
        mask, rot = d.get("mask"), d.get("rot")
        c = cls(heads, _get(d, "kv_heads", where, least=1, default=heads), dim,
                _get(d, "vdim", where, least=1, default=dim), _get(d, "scale", where, float),
                0 if mask is None else _get(mask, "size", where + ".mask", least=1),
                None if rot is None else RotaryTurn.from_dict(rot, where + ".rot", whole=dim),
                _get(d, "diff", where, float) if differential else None)
        if c.heads % c.kv_heads:
            raise ConfigError(f"config.json: '{where}.heads' ({c.heads}) is no multiple of kv_heads ({c.kv_heads})")
        return c

    def to_dict(self):
        d: Dict[str, Any] = {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "scale": self.scale,
                             "vdim": self.vdim}
        if self.window:
            d["mask"] = {"size": self.window}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        if self.diff is not None:
            d["diff"] = self.diff
        return d


@dataclass(frozen=True)
class SofinexFeedForward:
    kind: str  # "dense" | "moe"
    ff: int  # inner size (of an expert, for "moe")
    experts: int = 0  # experts with tensors
    identity: int = 0  # experts without: outputs of the router behind the others
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
                _get(router, "identity", w, least=0, default=0), _get(router, "top", w, least=1),
                0 if groups is None else _get(groups, "count", w + ".groups", least=1),
                0 if groups is None else _get(groups, "keep", w + ".groups", least=1),
                0 if shared is None else _get(shared, "ff", where + ".shared", least=1))
        n = c.experts + c.identity
        if c.top > n:
            raise ConfigError(f"config.json: '{w}.top' ({c.top}) is more than its {n} experts")
        if c.groups:
            if n % c.groups or c.keep > c.groups:
                raise ConfigError(f"config.json: '{w}.groups': {n} experts do not form {c.groups} equal groups of "
                                  f"which {c.keep} are kept")
            if c.keep * (n // c.groups) < c.top:
                raise ConfigError(f"config.json: '{w}.groups': {c.keep} groups of {n // c.groups} experts cannot "
                                  f"give {c.top} experts")
        return c

    def to_dict(self):
        if self.kind == "dense":
            return {"ff": self.ff, "kind": "dense"}
        router: Dict[str, Any] = {"experts": self.experts, "identity": self.identity, "top": self.top}
        if self.groups:
            router["groups"] = {"count": self.groups, "keep": self.keep}
        d: Dict[str, Any] = {"expert": {"ff": self.ff}, "kind": "moe", "router": router}
        if self.shared_ff:
            d["shared"] = {"ff": self.shared_ff}
        return d


@dataclass(frozen=True)
class SofinexLayer:
    type: str  # "attention" | "parallel"
    attention: Optional[WindowedHeads]  # type "attention": the differential mixer
    left: Optional[WindowedHeads]  # type "parallel"
    right: Optional[DeltaSide]
    mlp: Optional[SofinexFeedForward]

    @classmethod
    def from_dict(cls, d, i: int):
        where = f"layers[{i}]"
        if not isinstance(d, dict):
            raise ConfigError(f"config.json: '{where}' must be an object")
        kind, mixer, w = d.get("type"), d.get("mixer"), where + ".mixer"
        if kind not in ("attention", "parallel"):
            raise ConfigError(f"config.json: '{where}.type' must be 'attention' or 'parallel', found {kind!r}")
        if not isinstance(mixer, dict):
            raise ConfigError(f"config.json: required key '{w}' is missing")
        mlp = None if d.get("mlp") is None else SofinexFeedForward.from_dict(d["mlp"], where + ".mlp")
        if kind == "attention":
            return cls(kind, WindowedHeads.from_dict(mixer, w, True), None, None, mlp)
        return cls(kind, None, WindowedHeads.from_dict(mixer.get("left"), w + ".left", False),
                   DeltaSide.from_dict(mixer.get("right"), w + ".right"), mlp)

    def to_dict(self):
        mixer = self.attention.to_dict() if self.type == "attention" \
            else {"left": self.left.to_dict(), "right": self.right.to_dict()}
        return {"mixer": mixer, "mlp": None if self.mlp is None else self.mlp.to_dict(), "type": self.type}


@dataclass(frozen=True)
class SofinexConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    loop: Optional[Loop]
    layers: Tuple[SofinexLayer, ...]
    architecture: str = "Sofinex"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "SofinexConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        parsed = tuple(SofinexLayer.from_dict(x, i) for i, x in enumerate(layers))
        if not isinstance(d.get("norm"), dict):
            raise ConfigError("config.json: 'norm' must be an object")
        loop = None
        if d.get("loop") is not None:
            lp = d["loop"]
            loop = Loop(_get(lp, "start", "loop", least=0), _get(lp, "stop", "loop", least=0),
                        _get(lp, "times", "loop", least=1))
            if not loop.start <= loop.stop <= len(parsed):
                raise ConfigError(f"config.json: 'loop' runs layers {loop.start} to {loop.stop - 1} of {len(parsed)}")
        emb = d.get("embedding")
        return cls(vocab=_get(d, "vocab", "config", least=1), width=_get(d, "width", "config", least=1),
                   norm_eps=_get(d["norm"], "eps", "norm", float),
                   embedding_scale=1.0 if emb is None else _get(emb, "scale", "embedding", float, default=1.0),
                   loop=loop, layers=parsed, architecture=str(d.get("architecture", "Sofinex")))

    def run_order(self):
        """The layers in the order they run."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        lp = self.loop
        return list(range(lp.start)) + list(range(lp.start, lp.stop)) * lp.times + list(range(lp.stop, n))

    def completed(self, shapes: Mapping[str, Tuple[int, ...]]) -> "SofinexConfig":
        """The sizes that no key gives, from the shapes of a file's tensors (name -> shape)."""
        layers = list(self.layers)
        for i, layer in enumerate(layers):
            right = layer.right
            if right is None:
                continue
            for field, tensor in (("decay_rank", f"l{i}.mix.right.a1"), ("gate_rank", f"l{i}.mix.right.g1")):
                if getattr(right, field) is None:
                    shape = shapes.get(tensor)
                    if shape is None or len(shape) != 2:
                        raise ConfigError(f"layers[{i}]: the file has no matrix '{tensor}' to say the bottleneck's rank")
                    right = replace(right, **{field: int(shape[0])})
            layers[i] = replace(layer, right=right)
        return replace(self, layers=tuple(layers))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"architecture": self.architecture, "embedding": {"scale": self.embedding_scale},
                             "layers": [x.to_dict() for x in self.layers], "norm": {"eps": self.norm_eps},
                             "vocab": self.vocab, "width": self.width}
        if self.loop is not None:
            d["loop"] = self.loop.to_dict()
        return copy.deepcopy(d)
