"""Configurations, weights and the engine-beside-plain case for the Sofinex tests, shared by the CPU tests (the
engine's own code over the torch stand-in for the kernels) and the GPU tests (the same over the HIP kernels).
Every comparison is against `plain_sofinex`, run over whole sequences in float64.  The scenarios (cuttings,
batches, reuse of slots, long decoding, greedy tokens) are those of `vafodra_cases`, which ask nothing of a case
but its engine, its vocabulary and the plain logits."""
from __future__ import annotations

import copy
from typing import Dict, List, Optional

import torch

import longbow_quarrel_amd as lq
import plain_sofinex as ps
from vafodra_cases import (err, greedy, long_decoding, portions, slots_and_blocks_used_again, tokens,  # noqa: F401
                           unequal_batches, whole_and_token_by_token, write_folder)
from vupelorn_cases import assert_close_bf16  # noqa: F401
from longbow_quarrel_amd.engine import StepEntry

LLAMA = {"factor": 4.0, "original": 64, "low": 1.0, "high": 4.0}
YARN = {"factor": 6.0, "original": 48, "fast": 12.0, "slow": 1.5}


def _heads(heads, kv_heads, dim, vdim, scale, window=None, base=None, dims=None, scaling=None, diff=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window}
    if base is not None:
        m["rot"] = {"base": base, "dims": dim if dims is None else dims}
        if scaling is not None:
            m["rot"]["scaling"] = dict(scaling)
    if diff is not None:
        m["diff"] = diff
    return m


def _delta(heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "decay_rank": decay_rank,
            "gate_rank": gate_rank}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(experts, identity, top, ff, groups=None, shared=None):
    router = {"experts": experts, "identity": identity, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    d = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared is not None:
        d["shared"] = {"ff": shared}
    return d


def _diff_layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def _parallel(left, right, mlp):
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}


def _config(vocab, width, eps, emb_scale, layers, loop=None):
    d = {"architecture": "Sofinex", "embedding": {"scale": emb_scale}, "layers": layers, "norm": {"eps": eps},
         "vocab": vocab, "width": width}
    if loop is not None:
        d["loop"] = dict(zip(("start", "stop", "times"), loop))
    return d


# A: both kinds of layer; windows inside a cache block, across blocks and wider than any prompt here; keys wider and
# narrower than values; three query heads a kv head and one; rotations of a whole head and of a part, both scalings
# and none; delta heads that share q/k heads; ranks and taps that differ; identity experts (two, one, none), groups
# with one kept and all kept and none, a shared expert and none, a layer without feed-forward; the middle layers
# run three times
CFG_A = _config(173, 80, 1e-6, 3.0, [
    _parallel(_heads(6, 2, 24, 16, 0.3, 20, 3000.0, 16, YARN), _delta(4, 2, 12, 20, 4, 6, 10), _dense(56)),
    _diff_layer(_heads(2, 2, 16, 40, 0.25, 70, 500.0, 8, LLAMA, diff=0.65), _moe(4, 2, 2, 24, (3, 1), 40)),
    _parallel(_heads(4, 1, 32, 32, 0.15, 130, 10000.0, 8), _delta(3, 1, 16, 16, 3, 8, 8), None),
    _diff_layer(_heads(3, 1, 8, 24, 0.35, 1000, 100.0, None, {"factor": 2.0, "original": 16, "low": 2.0, "high": 8.0},
                       diff=0.3), _moe(5, 1, 3, 16, (2, 2))),
    _diff_layer(_heads(4, 2, 12, 12, 0.3, None, diff=0.8), _moe(3, 0, 1, 20, None, 12)),
], loop=(1, 3, 3))
# B: sizes that are multiples of nothing (the kernels' size-agnostic ways), one head, a window of one token, all
# experts chosen, more identity experts than others, a loop that is the whole model run twice, an embedding as it is
CFG_B = _config(97, 50, 1e-5, 1.0, [
    _diff_layer(_heads(1, 1, 10, 7, 0.4, 5, 250.0, 6, diff=0.45), _moe(1, 3, 2, 9, (2, 1), 11)),
    _parallel(_heads(5, 5, 6, 10, 0.5, 1), _delta(2, 1, 5, 7, 2, 1, 1), _dense(21)),
    _parallel(_heads(2, 1, 14, 14, 0.25, 64, 1000.0, None, {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 2.0}),
              _delta(3, 3, 7, 3, 5, 2, 7), _moe(2, 1, 3, 13)),
], loop=(0, 3, 2))
# C: head sizes, ranks and widths of the kind that the fast kernels are made for; no loop
CFG_C = _config(1000, 320, 1e-5, 8.0, [
    _parallel(_heads(4, 2, 64, 32, 0.12, 100, 10000.0, 32, {"factor": 4.0, "original": 128, "fast": 32.0, "slow": 1.0}),
              _delta(4, 2, 32, 64, 4, 16, 32), _moe(6, 2, 2, 64, (4, 2), 192)),
    _diff_layer(_heads(8, 2, 32, 64, 0.18, 65, 40000.0, 16, {"factor": 8.0, "original": 256, "low": 1.0, "high": 4.0},
                       diff=0.7), _dense(384)),
    _diff_layer(_heads(2, 1, 128, 128, 0.09, 200, 10000.0, 64, diff=0.5), _moe(4, 0, 1, 128, None, 64)),
    _parallel(_heads(8, 8, 32, 64, 0.18, 63, 40000.0), _delta(8, 8, 16, 16, 2, 8, 8), None),
])
# one mechanism a model: what fails here names its mechanism
CFG_DIFF = _config(60, 48, 1e-6, 2.0, [
    _diff_layer(_heads(4, 2, 16, 8, 0.3, 40, 200.0, 12, {"factor": 3.0, "original": 20, "low": 1.0, "high": 5.0},
                       diff=0.55), None)])
CFG_SINK = _config(60, 48, 1e-6, 2.0, [
    _parallel(_heads(4, 2, 16, 8, 0.3, 40, 200.0, 12, {"factor": 3.0, "original": 20, "fast": 8.0, "slow": 1.0}),
              _delta(1, 1, 8, 8, 2, 2, 2), None)])
CFG_DELTA = _config(60, 48, 1e-6, 2.0, [
    _parallel(_heads(1, 1, 8, 8, 0.3, 3), _delta(4, 2, 12, 20, 3, 5, 7), None)])
CFG_DENSE = _config(60, 48, 1e-6, 2.0, [
    _diff_layer(_heads(1, 1, 8, 8, 0.3, 10, 100.0, diff=0.5), _dense(40))])
CFG_MOE = _config(60, 48, 1e-6, 2.0, [
    _diff_layer(_heads(1, 1, 8, 8, 0.3, 10, 100.0, diff=0.5), _moe(9, 3, 3, 20, (4, 2), 28))])
CFG_LOOP = _config(60, 48, 1e-6, 1.5, [
    _parallel(_heads(2, 1, 8, 8, 0.3, 30, 100.0), _delta(1, 1, 8, 8, 2, 2, 2), _dense(24)),
    _diff_layer(_heads(1, 1, 16, 8, 0.2, 25, 100.0, diff=0.65), None),
    _parallel(_heads(2, 2, 8, 16, 0.3, 66, 100.0), _delta(2, 1, 8, 8, 2, 3, 3), _dense(16)),
], loop=(0, 2, 3))
CONFIGS = {"a": CFG_A, "b": CFG_B, "c": CFG_C, "diff": CFG_DIFF, "sink": CFG_SINK, "delta": CFG_DELTA,
           "dense": CFG_DENSE, "moe": CFG_MOE, "loop": CFG_LOOP}


def windowed(kind: str, window: int) -> dict:
    """One attention layer of the kind ("diff" or "sink") with the window given."""
    cfg = copy.deepcopy(CFG_DIFF if kind == "diff" else CFG_SINK)
    mixer = cfg["layers"][0]["mixer"]
    (mixer if kind == "diff" else mixer["left"])["mask"]["size"] = window
    return cfg


def random_config(seed: int) -> dict:
    """A configuration drawn from a seed: the layers' kinds and order, sizes, head counts, windows, rotations, ranks,
    the feed-forwards, the loop and the constants all vary; some sizes are multiples of 16, some of nothing."""
    import random

    rng = random.Random(seed)
    width = rng.choice([40, 56, 64, 72, 100, 128, 136])

    def heads(diff):
        kv = rng.randint(1, 3)
        dim = rng.choice([8, 12, 16, 20, 32, 48, 64])
        base = rng.choice([None, 100.0, 10000.0, 250000.0])
        scaling = None
        if base is not None and rng.random() < 0.7:
            scaling = {"factor": rng.choice([2.0, 4.0, 8.0]), "original": rng.choice([16, 64, 2048])}
            if rng.random() < 0.5:
                scaling.update(fast=rng.choice([8.0, 32.0]), slow=rng.choice([1.0, 2.0]))
            else:
                scaling.update(low=rng.choice([1.0, 2.0]), high=rng.choice([4.0, 8.0]))
        return _heads(kv * rng.randint(1, 3), kv, dim, rng.choice([8, 16, 28, 64]), rng.choice([0.1, 0.2, 0.35]),
                      rng.choice([None, 1, 2, 7, 33, 64, 65, 100]), base,
                      None if base is None or rng.random() < 0.5 else 2 * rng.randint(1, dim // 2), scaling,
                      rng.choice([0.2, 0.5, 0.8]) if diff else None)

    layers = []
    for _ in range(rng.randint(1, 5)):
        kind = rng.choice(["none", "dense", "moe", "moe"])
        mlp = None
        if kind == "dense":
            mlp = _dense(rng.choice([16, 24, 50, 96]))
        elif kind == "moe":
            groups = rng.choice([None, (2, 1), (2, 2), (3, 2), (4, 3)])
            per = rng.randint(1, 3)
            outputs = per * groups[0] if groups else rng.randint(2, 8)
            identity = rng.randint(0, outputs - 1)
            most = groups[1] * per if groups else outputs
            mlp = _moe(outputs - identity, identity, rng.randint(1, most), rng.choice([8, 12, 20, 32]), groups,
                       rng.choice([None, 8, 24, 36]))
        if rng.random() < 0.5:
            layers.append(_diff_layer(heads(True), mlp))
        else:
            rkv = rng.randint(1, 2)
            right = _delta(rkv * rng.randint(1, 3), rkv, rng.choice([8, 12, 16, 24, 40]), rng.choice([8, 12, 16, 36]),
                           rng.randint(1, 5), rng.randint(1, 9), rng.randint(1, 9))
            layers.append(_parallel(heads(False), right, mlp))
    loop = None
    if rng.random() < 0.7:
        start = rng.randint(0, len(layers) - 1)
        loop = (start, rng.randint(start, len(layers)), rng.randint(1, 3))
    return _config(rng.randint(30, 300), width, rng.choice([1e-6, 1e-5]), rng.choice([1.0, 2.5, 12.0]), layers, loop)


def make_weights(cfg: dict, seed: int, sharp: float = 1.0, memory: float = 0.0) -> Dict[str, torch.Tensor]:
    """Random weights whose values bfloat16 holds exactly (both run dtypes then see the same model), with spreads
    that make every constant matter.  `sharp` multiplies the attention's score scales in `cfg` (in place) so that
    attention is peaked.  `memory` is subtracted from the decays' biases, so that a delta-rule state forgets slowly
    and old tokens stay in it."""
    from longbow_quarrel_amd.model import DecoderModel
    from longbow_quarrel_amd.registry import spec_from_config

    if sharp != 1.0:
        for layer in cfg["layers"]:
            m = layer["mixer"]
            (m if layer["type"] == "attention" else m["left"])["scale"] *= sharp
    config = lq.SofinexConfig.from_dict(cfg)
    g = torch.Generator().manual_seed(seed)
    out = {}
    for s in DecoderModel(spec_from_config(config)).tensor_specs():
        n, shape = s.name, tuple(s.shape)
        leaf = n.split(".")[-1]
        normal = lambda std, mean=0.0: torch.empty(shape).normal_(mean, std, generator=g)
        if n == "embed":
            t = normal(0.5)
        elif leaf in ("norm1", "norm2") or n == "final.norm":  # gains stored around zero
            t = normal(0.3)
        elif leaf in ("norm", "out"):
            t = normal(0.3, 1.0)
        elif leaf == "conv":
            t = normal(0.6)
        elif leaf == "A_log":
            t = normal(0.5, -0.5)
        elif leaf == "dt_bias":
            t = normal(1.0, -memory)
        elif leaf == "correction":
            t = normal(0.15)
        elif leaf == "sink":
            t = normal(1.0)
        elif leaf in ("lq1", "lk1", "lq2", "lk2"):
            t = normal(0.5)
        elif leaf in ("router", "sg"):
            t = normal(2.0 / (shape[-1] ** 0.5))
        else:
            t = normal(1.0 / (shape[-1] ** 0.5))
        out[n] = t.to(torch.bfloat16).float()
    return out


class Case:
    """An engine (made by `load`, which the CPU and the GPU tests bring) beside the plain implementation."""

    def __init__(self, tmp_path, name, load, dtype: str = "float32", seed: int = 3, sharp: float = 1.0,
                 memory: float = 0.0, max_tokens: int = 2048, rounding: bool = False,
                 cfg: Optional[dict] = None) -> None:
        self.cfg = copy.deepcopy(cfg if cfg is not None else CONFIGS[name] if isinstance(name, str)
                                 else random_config(name))
        self.weights = make_weights(self.cfg, seed, sharp, memory)
        self.folder = write_folder(tmp_path, self.cfg, self.weights, f"{name}_{seed}_{sharp}_{memory}")
        self.eng = load(self.folder, dtype, max_tokens)
        self.vocab = self.cfg["vocab"]
        self.rounding = rounding
        self._want = {}

    def want(self, toks: List[int]) -> torch.Tensor:
        key = tuple(toks)
        if key not in self._want:
            self._want[key] = ps.forward(self.cfg, self.weights, toks, rounding=self.rounding)
        return self._want[key]

    def noise(self, toks: List[int]) -> float:
        """What rounding alone does on these tokens: the median over the rows of the largest difference (over the
        largest logit) between the plain implementation with and without rounding."""
        a = ps.forward(self.cfg, self.weights, toks, rounding=True)
        b = ps.forward(self.cfg, self.weights, toks, rounding=False)
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
        ps.forward(self.cfg, self.weights, toks, rounding=self.rounding, layers_out=want)
        return got, want

    def assert_idle(self) -> None:
        c = self.eng.cache
        assert c.slots.taken_count == 0 and all(g.blocks.taken_count == 0 for g in c.kv_groups)


def a_window_off_by_one_would_show(case: Case, toks: List[int], kind: str, rows) -> None:
    """The plain implementation with the window a token wider and a token narrower differs from the true one at
    `rows` by much more than any tolerance here: were the engine's window off by one, the comparison would fail."""
    for other in (+1, -1):
        cfg = copy.deepcopy(case.cfg)
        mixer = cfg["layers"][0]["mixer"]
        mask = (mixer if kind == "diff" else mixer["left"])["mask"]
        if mask["size"] + other < 1:
            continue
        mask["size"] += other
        wrong = ps.forward(cfg, case.weights, toks)
        assert err(wrong[rows], case.want(toks)[rows]) > 1e-3, f"a window off by {other} does not show"
