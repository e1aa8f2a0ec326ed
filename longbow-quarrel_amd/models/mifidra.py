"""The Mifidra decoder as a `ModelSpec`.

Every layer has a norm ahead of each sublayer and one on its result: x += norm1b(mixer(norm1(x)));
x += norm2b(ffn(norm2(x))).  The mixer is two mixers side by side on the same input, their results added with a
constant each: causal softmax attention (grouped key/value heads; interleaved rotary pairs on the first entries of
every head under YaRN scaling; q and k divided by their root mean square after the rotation) and the gated delta rule
with a decay for every key channel and a sigmoid gate, both through bottlenecks.  The feed-forward is a gated unit with
biases, or a mixture of experts chosen by sigmoid scores with a correction, within the best groups, beside a shared
expert.  A stretch of the layers may run several times in a row with the same weights (every run a cache of its own);
the embedding's output is added to the stream ahead of every pass but the first.  The head is the embedding, and the
logits are scaled.

Tensor names: `embed`, `final.norm`, and for layer i `l<i>.norm1`, `l<i>.norm1b`, `l<i>.norm2`, `l<i>.norm2b`,
`l<i>.mix.left.*`, `l<i>.mix.right.*`, `l<i>.mlp.*`.
"""
from __future__ import annotations

from ..config.base import ConfigError
from ..config.mifidra import MifidraConfig, MifidraLayer
from ..model import ModelSpec, Run, token_table
from ..parts.base import PartSpec
from ..registry import register_architecture


def _mixer(cfg: MifidraConfig, layer: MifidraLayer, i: int) -> PartSpec:
    prefix = f"l{i}.mix"
    a, r = layer.left, layer.right
    rotary = None
    if a.rot is not None:
        scaling = None
        if a.rot.scaling is not None:
            sc = a.rot.scaling
            scaling = {"rope_type": "yarn", "factor": sc.factor, "original": sc.original, "fast": sc.fast,
                       "slow": sc.slow}
        rotary = {"dims": a.rot.dims, "base": a.rot.base, "scaling": scaling, "pairing": "interleaved"}
    left = PartSpec("sink_window_attention", {
        "width": cfg.width, "heads": a.heads, "kv_heads": a.kv_heads, "key_dim": a.dim, "value_dim": a.vdim,
        "scale": a.scale, "window": 0, "keep_first": 0, "sink": False, "head_gate": False, "rotary": rotary,
        "qk_norm_eps": cfg.norm_eps, "prefix": prefix + ".left"})
    if r.decay_rank is None or r.gate_rank is None:
        raise ConfigError(f"layers[{i}].mixer.right: the bottlenecks' ranks are in no key; a model file's tensor "
                          "shapes give them (or state 'decay_rank' and 'gate_rank')")
    right = PartSpec("gated_delta", {
        "width": cfg.width, "heads": r.heads, "kv_heads": r.kv_heads, "key_dim": r.dim, "value_dim": r.vdim,
        "conv": r.conv, "eps": cfg.norm_eps, "decay": "channel", "decay_rank": r.decay_rank, "gate": "sigmoid",
        "gate_rank": r.gate_rank, "prefix": prefix + ".right"})
    return PartSpec("side_by_side", {"width": cfg.width, "eps": cfg.norm_eps, "sides": (left, right),
                                     "weights": (layer.left_scale, layer.right_scale)})


def _feed_forward(cfg: MifidraConfig, layer: MifidraLayer, i: int):
    m = layer.mlp
    if m is None:
        return None
    if m.kind == "dense":
        return PartSpec("glu", {"width": cfg.width, "inner": m.ff, "prefix": f"l{i}.mlp", "activation": "silu",
                                "bias": True})
    return PartSpec("moe", {"width": cfg.width, "experts": m.experts, "top": m.top, "inner": m.ff,
                            "prefix": f"l{i}.mlp", "weight_input": False, "renormalize": False, "activation": "silu",
                            "correction": True, "groups": m.groups, "keep": m.keep, "shared_inner": m.shared_ff})


def mifidra_spec(cfg: MifidraConfig) -> ModelSpec:
    def norm(name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"width": cfg.width, "eps": cfg.norm_eps, "name": name})

    blocks = []
    for i, layer in enumerate(cfg.layers):
        ffn = _feed_forward(cfg, layer, i)
        blocks.append(PartSpec("sandwich_norm", {
            "mixer": _mixer(cfg, layer, i), "mixer_norm": norm(f"l{i}.norm1"), "mixer_out_norm": norm(f"l{i}.norm1b"),
            "feed_forward": ffn, "ffn_norm": norm(f"l{i}.norm2"), "ffn_out_norm": norm(f"l{i}.norm2b")}))
    schedule = tuple(Run(i, add_input=again) for i, again in cfg.run_order())
    return ModelSpec(
        vocab_size=cfg.vocab, width=cfg.width, embedding=token_table("embed", cfg.vocab, cfg.width),
        layers=tuple(blocks), schedule=schedule, final_norm=norm("final.norm"), head_name=None, tie_head=True,
        logits_step=None if cfg.logit_scale == 1.0 else PartSpec("scale", {"factor": cfg.logit_scale}),
        max_positions=None,  # nothing in the design depends on a longest sequence
    )


register_architecture("Mifidra", MifidraConfig, mifidra_spec)
