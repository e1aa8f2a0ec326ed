"""Configurations, weights and the engine-beside-plain case for the Mifidra tests, shared by the CPU tests (the
engine's own code over the torch stand-in for the kernels) and the GPU tests (the same over the HIP kernels).
Every comparison is against `plain_mifidra`, run over whole sequences in float64.  The scenarios (cuttings,
batches, reuse of slots, long decoding, greedy tokens) are those of `vafodra_cases`, which ask nothing of a case
but its engine, its vocabulary and the plain logits."""
from __future__ import annotations

import copy
from typing import Dict, List

import torch

import longbow_quarrel_amd as lq
import plain_mifidra as pm
from vafodra_cases import (err, greedy, long_decoding, portions, slots_and_blocks_used_again, tokens,  # noqa: F401
                           unequal_batches, whole_and_token_by_token, write_folder)
from vupelorn_cases import assert_close_bf16  # noqa: F401
from longbow_quarrel_amd.engine import StepEntry


def _left(heads, kv_heads, dim, vdim, scale, base=None, dims=None, scaling=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if base is not None:
        m["rot"] = {"base": base, "dims": dim if dims is None else dims}
        if scaling is not None:
            m["rot"]["scaling"] = scaling
    return m


def _right(heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "decay_rank": decay_rank,
            "gate_rank": gate_rank}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, top, ff, groups=None, shared=None):
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    d = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        d["shared"] = {"ff": shared}
    return d


def _layer(left, right, left_scale, right_scale, mlp):
    return {"type": "parallel", "mixer": {"left": left, "left_scale": left_scale, "right": right,
                                          "right_scale": right_scale}, "mlp": mlp}


def _config(vocab, width, eps, logit_scale, layers, loop=None):
    d = {"architecture": "Mifidra", "layers": layers, "logit_scale": logit_scale, "norm": {"eps": eps},
         "vocab": vocab, "width": width}
    if loop is not None:
        d["loop"] = dict(zip(("start", "stop", "times"), loop))
    return d


_YARN = {"factor": 6.0, "original": 48, "fast": 12.0, "slow": 1.5}
# A: keys wider than values and narrower, a rotation of fewer entries than a head holds, three query heads a kv head
# and one, delta heads that share q/k heads, ranks that differ, convolutions of 4 and 2 taps, a dense layer, experts
# in groups with a shared expert, experts without groups or shared expert, a layer without feed-forward; the middle
# layers run three times
CFG_A = _config(173, 80, 1e-6, 0.7, [
    _layer(_left(6, 2, 24, 16, 0.3, 3000.0, 16, _YARN), _right(4, 2, 12, 20, 4, 6, 10), 0.6, 1.3, _dense(56)),
    _layer(_left(2, 2, 16, 40, 0.2, 500.0), _right(2, 2, 20, 8, 2, 3, 5), 1.1, 0.4, _moe(6, 2, 24, (3, 2), 40)),
    _layer(_left(4, 1, 32, 32, 0.15, 10000.0, 8), _right(3, 1, 16, 16, 3, 8, 8), 0.9, 0.8, None),
    _layer(_left(3, 3, 8, 24, 0.35, 100.0, scaling={"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0}),
           _right(1, 1, 40, 24, 1, 4, 2), 1.0, 1.0, _moe(4, 3, 16)),
], loop=(1, 3, 3))
# B: sizes that are multiples of nothing (the kernels' size-agnostic ways), one head, no rotation in one layer, all
# experts chosen, one group kept of two, a loop that is the whole model run twice, logits as they are
CFG_B = _config(97, 50, 1e-5, 1.0, [
    _layer(_left(1, 1, 10, 7, 0.4, 250.0, 6), _right(1, 1, 9, 13, 3, 5, 3), 1.2, 0.7, _moe(4, 2, 9, (2, 1), 11)),
    _layer(_left(5, 5, 6, 10, 0.5), _right(2, 1, 5, 7, 2, 1, 1), 0.5, 1.5, _dense(21)),
    _layer(_left(2, 1, 14, 14, 0.25, 1000.0, scaling={"factor": 4.0, "original": 32, "fast": 8.0, "slow": 2.0}),
           _right(3, 3, 7, 3, 5, 2, 7), 0.8, 0.9, _moe(3, 3, 13)),
], loop=(0, 3, 2))
# C: head sizes, ranks and widths of the kind that the fast kernels are made for; no loop
CFG_C = _config(1000, 320, 1e-5, 0.25, [
    _layer(_left(4, 2, 64, 32, 0.12, 10000.0, 32, {"factor": 4.0, "original": 128, "fast": 32.0, "slow": 1.0}),
           _right(4, 2, 32, 64, 4, 16, 32), 0.7, 1.1, _moe(8, 2, 64, (4, 2), 192)),
    _layer(_left(8, 8, 32, 64, 0.18, 40000.0), _right(2, 1, 64, 32, 3, 32, 16), 1.0, 0.5, _dense(384)),
    _layer(_left(2, 1, 128, 128, 0.09, 10000.0, 64), _right(8, 8, 16, 16, 2, 8, 8), 0.9, 0.9, _moe(4, 1, 128, None, 64)),
])
# D: attention heads whose keys and values are of one size that the causal matrix-core kernel takes (a bfloat16 run
# then goes through it, a float32 run through the general kernel)
CFG_D = _config(500, 256, 1e-5, 0.5, [
    _layer(_left(8, 2, 64, 64, 0.125, 10000.0, 32, {"factor": 4.0, "original": 128, "fast": 32.0, "slow": 1.0}),
           _right(2, 1, 32, 32, 4, 16, 16), 0.8, 0.9, _dense(384)),
    _layer(_left(4, 4, 128, 128, 0.09, 40000.0), _right(2, 2, 16, 64, 3, 8, 16), 1.0, 0.5, _moe(8, 2, 64, (4, 2), 128)),
    _layer(_left(6, 1, 32, 32, 0.18, 10000.0, 16), _right(4, 2, 32, 16, 2, 8, 8), 0.9, 1.1, None),
], loop=(0, 2, 2))
# one mechanism a model: what fails here names its mechanism (the other side of the mixer is weighted with zero)
CFG_ATTENTION = _config(60, 48, 1e-6, 1.0, [
    _layer(_left(4, 2, 16, 8, 0.3, 200.0, 12, {"factor": 3.0, "original": 20, "fast": 8.0, "slow": 1.0}),
           _right(1, 1, 8, 8, 2, 2, 2), 1.0, 0.0, None)])
CFG_DELTA = _config(60, 48, 1e-6, 1.0, [
    _layer(_left(1, 1, 8, 8, 0.3), _right(4, 2, 12, 20, 3, 5, 7), 0.0, 1.0, None)])
CFG_DENSE = _config(60, 48, 1e-6, 1.0, [
    _layer(_left(1, 1, 8, 8, 0.3, 100.0), _right(1, 1, 8, 8, 2, 2, 2), 0.5, 0.5, _dense(40))])
CFG_MOE = _config(60, 48, 1e-6, 1.0, [
    _layer(_left(1, 1, 8, 8, 0.3, 100.0), _right(1, 1, 8, 8, 2, 2, 2), 0.5, 0.5, _moe(12, 3, 20, (4, 2), 28))])
CFG_LOOP = _config(60, 48, 1e-6, 2.0, [
    _layer(_left(2, 1, 8, 8, 0.3, 100.0), _right(1, 1, 8, 8, 2, 2, 2), 0.8, 0.6, _dense(24)),
    _layer(_left(1, 1, 16, 8, 0.2, 100.0), _right(2, 2, 8, 8, 3, 2, 2), 0.7, 0.9, None),
    _layer(_left(2, 2, 8, 16, 0.3, 100.0), _right(2, 1, 8, 8, 2, 3, 3), 0.6, 0.8, _dense(16)),
], loop=(0, 2, 3))
CONFIGS = {"a": CFG_A, "b": CFG_B, "c": CFG_C, "d": CFG_D, "attention": CFG_ATTENTION, "delta": CFG_DELTA, "dense": CFG_DENSE,
           "moe": CFG_MOE, "loop": CFG_LOOP}


def random_config(seed: int) -> dict:
    """A configuration drawn from a seed: sizes, head counts, ranks, the feed-forwards, the loop and the constants
    all vary; some sizes are multiples of 16, some of nothing."""
    import random

    rng = random.Random(seed)
    width = rng.choice([40, 56, 64, 72, 100, 128, 136])
    layers = []
    for _ in range(rng.randint(1, 5)):
        kv = rng.randint(1, 3)
        dim = rng.choice([8, 12, 16, 20, 32, 48, 64])
        base = rng.choice([None, 100.0, 10000.0, 250000.0])
        scaling = None
        if base is not None and rng.random() < 0.6:
            scaling = {"factor": rng.choice([2.0, 4.0, 8.0]), "original": rng.choice([16, 64, 2048]),
                       "fast": rng.choice([8.0, 32.0]), "slow": rng.choice([1.0, 2.0])}
        left = _left(kv * rng.randint(1, 3), kv, dim, rng.choice([8, 16, 28, 64]), rng.choice([0.1, 0.2, 0.35]), base,
                     None if base is None or rng.random() < 0.5 else 2 * rng.randint(1, dim // 2), scaling)
        rkv = rng.randint(1, 2)
        right = _right(rkv * rng.randint(1, 3), rkv, rng.choice([8, 12, 16, 24, 40]), rng.choice([8, 12, 16, 36]),
                       rng.randint(1, 5), rng.randint(1, 9), rng.randint(1, 9))
        kind = rng.choice(["none", "dense", "moe", "moe"])
        mlp = None
        if kind == "dense":
            mlp = _dense(rng.choice([16, 24, 50, 96]))
        elif kind == "moe":
            groups = rng.choice([None, (2, 1), (2, 2), (3, 2), (4, 3)])
            per = rng.randint(1, 3)
            experts = per * groups[0] if groups else rng.randint(2, 8)
            most = groups[1] * per if groups else experts
            mlp = _moe(experts, rng.randint(1, most), rng.choice([8, 12, 20, 32]), groups,
                       rng.choice([None, 8, 24, 36]))
        layers.append(_layer(left, right, rng.choice([0.5, 0.8, 1.0, 1.25]), rng.choice([0.5, 0.9, 1.0, 1.5]), mlp))
    loop = None
    if rng.random() < 0.7:
        start = rng.randint(0, len(layers) - 1)
        loop = (start, rng.randint(start, len(layers)), rng.randint(1, 3))
    return _config(rng.randint(30, 300), width, rng.choice([1e-6, 1e-5]), rng.choice([0.5, 1.0, 3.0]), layers, loop)


def make_weights(cfg: dict, seed: int, sharp: float = 1.0, memory: float = 0.0) -> Dict[str, torch.Tensor]:
    """Random weights whose values bfloat16 holds exactly (both run dtypes then see the same model), with spreads
    that make every constant matter.  `sharp` multiplies the attention's score scale in `cfg` (in place) so that
    attention is peaked: q and k are unit-normed, so only the scale can sharpen it.  `memory` is subtracted from the
    decays' biases, so that a delta-rule state forgets slowly and old tokens stay in it."""
    config = lq.MifidraConfig.from_dict(cfg)
    from longbow_quarrel_amd.model import DecoderModel
    from longbow_quarrel_amd.registry import spec_from_config

    if sharp != 1.0:
        for layer in cfg["layers"]:
            layer["mixer"]["left"]["scale"] *= sharp
        config = lq.MifidraConfig.from_dict(cfg)
    g = torch.Generator().manual_seed(seed)
    out = {}
    for s in DecoderModel(spec_from_config(config)).tensor_specs():
        n, shape = s.name, tuple(s.shape)
        leaf = n.split(".")[-1]
        normal = lambda std, mean=0.0: torch.empty(shape).normal_(mean, std, generator=g)
        if n == "embed":
            t = normal(0.5)
        elif leaf in ("norm", "norm1", "norm2", "norm1b", "norm2b") or n == "final.norm":
            t = normal(0.3, 1.0)
        elif leaf == "conv":
            t = normal(0.6)
        elif leaf == "A_log":
            t = normal(0.5, -0.5)
        elif leaf == "dt_bias":
            t = normal(1.0, -memory)
        elif leaf == "correction":
            t = normal(0.3)
        elif leaf == "b" and len(shape) == 1:  # a feed-forward's bias
            t = normal(0.3)
        elif leaf == "router":  # (scores well inside (0, 1))
            t = normal(0.5 / (shape[-1] ** 0.5))
        else:
            t = normal(1.0 / (shape[-1] ** 0.5))
        out[n] = t.to(torch.bfloat16).float()
    return out


class Case:
    """An engine (made by `load`, which the CPU and the GPU tests bring) beside the plain implementation."""

    def __init__(self, tmp_path, name, load, dtype: str = "float32", seed: int = 3, sharp: float = 1.0,
                 memory: float = 0.0, max_tokens: int = 2048, rounding: bool = False) -> None:
        self.cfg = copy.deepcopy(CONFIGS[name] if isinstance(name, str) else random_config(name))
        self.weights = make_weights(self.cfg, seed, sharp, memory)
        self.folder = write_folder(tmp_path, self.cfg, self.weights, f"{name}_{seed}_{sharp}_{memory}")
        self.eng = load(self.folder, dtype, max_tokens)
        self.vocab = self.cfg["vocab"]
        self.rounding = rounding
        self._want = {}

    def want(self, toks: List[int]) -> torch.Tensor:
        key = tuple(toks)
        if key not in self._want:
            self._want[key] = pm.forward(self.cfg, self.weights, toks, rounding=self.rounding)
        return self._want[key]

    def noise(self, toks: List[int]) -> float:
        """What rounding alone does on these tokens: the median over the rows of the largest difference (over the
        largest logit) between the plain implementation with and without rounding."""
        a = pm.forward(self.cfg, self.weights, toks, rounding=True)
        b = pm.forward(self.cfg, self.weights, toks, rounding=False)
        return float(((a - b).abs().max(-1).values / b.abs().max()).median())

    def run_cut(self, toks: List[int], cuts: List[int]) -> torch.Tensor:
        """The sequence in portions of the sizes `cuts` (the rest token by token), all logits."""
        eng = self.eng
        s = eng.new_sequence()
        got, at = [], 0
        sizes = list(cuts)
        while at < len(toks):
            n = min(sizes.pop(0) if sizes else 1, len(toks) - at)
            got.append(eng.step([StepEntry(s, toks[at : at + n], range(n))]).clone())
            at += n
        eng.release(s)
        return torch.cat(got)

    def layers(self, toks: List[int]):
        """The residual stream after every layer run, from the engine's observer and from the plain implementation."""
        got = []

        def see(name, x, pending):
            if name != "embed":
                full = x.float().cpu().clone()
                if pending is not None:
                    full += pending.float().cpu().sum(0) if pending.dim() == 3 else pending.float().cpu()
                got.append(full)

        s = self.eng.new_sequence()
        self.eng.step([StepEntry(s, toks, [])], observe=see)
        self.eng.release(s)
        want = []
        pm.forward(self.cfg, self.weights, toks, rounding=self.rounding, layers_out=want)
        return got, want

    def assert_idle(self) -> None:
        c = self.eng.cache
        assert c.slots.taken_count == 0 and all(g.blocks.taken_count == 0 for g in c.kv_groups)
