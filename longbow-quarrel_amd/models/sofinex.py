"""The Sofinex decoder as a `ModelSpec`.

Every layer is a pre-norm block, x += mixer(N1(x)); x += ffn(N2(x)), whose norms store their gains around zero
(N(x) = x / rms(x) (1 + w)).  An "attention" layer's mixer is differential attention under a sliding window; a
"parallel" layer's mixer is windowed softmax attention (half-split rotary pairs under YaRN scaling, q and k divided by
their root mean square after the rotation, a learned sink a head) beside the gated delta rule with a decay for every
key channel and a sigmoid gate, each result RMS-normed over the width with a weight of its own, half their sum.  The
feed-forward is two matrices around the exact gelu, or a mixture of experts: softmax scores, the choice by score plus
a stored correction within the groups whose best choice score is highest, the chosen scores renormalised, identity
experts among the router's outputs, and a shared expert behind a sigmoid gate a token; a layer may have none.  A
stretch of the layers may run several times in a row with the same weights (every run a cache of its own).  The
embedding is scaled, and the head is a matrix of its own.

Tensor names: `embed`, `head`, `final.norm`, and for layer i `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.*` (a parallel
layer's under `.left` and `.right`, its output weights `l<i>.mix.left.out` and `.right.out`), `l<i>.mlp.*`.
"""
from __future__ import annotations

from ..config.base import ConfigError
from ..config.sofinex import SofinexConfig, SofinexLayer
from ..model import ModelSpec, Run, token_table
from ..parts.base import PartSpec
from ..registry import register_architecture

#: what the chosen scores' sum is raised by before the weights are divided by it
RENORMALIZE_EPS = 1e-20


def _mixer(cfg: SofinexConfig, layer: SofinexLayer, i: int) -> PartSpec:
    prefix = f"l{i}.mix"
    if layer.type == "attention":
        a = layer.attention
        return PartSpec("differential_attention", {
            "width": cfg.width, "heads": a.heads, "kv_heads": a.kv_heads, "key_dim": a.dim, "value_dim": a.vdim,
            "scale": a.scale, "diff": a.diff, "eps": cfg.norm_eps, "window": a.window,
            "rotary": None if a.rot is None else a.rot.as_parameters(), "prefix": prefix})
    a, r = layer.left, layer.right
    left = PartSpec("sink_window_attention", {
        "width": cfg.width, "heads": a.heads, "kv_heads": a.kv_heads, "key_dim": a.dim, "value_dim": a.vdim,
        "scale": a.scale, "window": a.window, "keep_first": 0, "sink": "learned", "head_gate": False,
        "rotary": None if a.rot is None else a.rot.as_parameters(), "qk_norm_eps": cfg.norm_eps,
        "prefix": prefix + ".left"})
    if r.decay_rank is None or r.gate_rank is None:
        raise ConfigError(f"layers[{i}].mixer.right: the bottlenecks' ranks are in no key; a model file's tensor "
                          "shapes give them (or state 'decay_rank' and 'gate_rank')")
    right = PartSpec("gated_delta", {
        "width": cfg.width, "heads": r.heads, "kv_heads": r.kv_heads, "key_dim": r.dim, "value_dim": r.vdim,
        "conv": r.conv, "eps": cfg.norm_eps, "decay": "channel", "decay_rank": r.decay_rank, "gate": "sigmoid",
        "gate_rank": r.gate_rank, "prefix": prefix + ".right"})
    return PartSpec("side_by_side", {"width": cfg.width, "eps": cfg.norm_eps, "sides": (left, right),
                                     "out_names": (prefix + ".left.out", prefix + ".right.out")})


def _feed_forward(cfg: SofinexConfig, layer: SofinexLayer, i: int):
    m = layer.mlp
    if m is None:
        return None
    if m.kind == "dense":
        return PartSpec("mlp", {"width": cfg.width, "inner": m.ff, "prefix": f"l{i}.mlp", "activation": "gelu"})
    return PartSpec("moe", {"width": cfg.width, "experts": m.experts, "top": m.top, "inner": m.ff,
                            "prefix": f"l{i}.mlp", "weight_input": False, "renormalize": True,
                            "renormalize_eps": RENORMALIZE_EPS, "activation": "silu", "scoring": "softmax",
                            "correction": True, "groups": m.groups, "keep": m.keep, "group_mark": "max",
                            "identity": m.identity, "shared_inner": m.shared_ff, "shared_gate": bool(m.shared_ff)})


def sofinex_spec(cfg: SofinexConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.norm_eps, "name": name, "offset": 1.0})

    blocks = [PartSpec("prenorm", {"mixer": _mixer(cfg, layer, i), "mixer_norm": norm(f"l{i}.norm1"),
                                   "feed_forward": _feed_forward(cfg, layer, i), "ffn_norm": norm(f"l{i}.norm2")})
              for i, layer in enumerate(cfg.layers)]
    return ModelSpec(
        vocab_size=cfg.vocab, width=cfg.width,
        embedding=token_table("embed", cfg.vocab, cfg.width, scale=cfg.embedding_scale),
        layers=tuple(blocks), schedule=tuple(Run(i) for i in cfg.run_order()), final_norm=norm("final.norm"),
        head_name="head", tie_head=False,
        max_positions=None,  # nothing in the design depends on a longest sequence
    )


register_architecture("Sofinex", SofinexConfig, sofinex_spec)
