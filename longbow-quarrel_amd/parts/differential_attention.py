"""Differential attention (Ye, Dong, Xia, Sun, Zhu, Huang, Wei: "Differential Transformer"): every query head
asks twice, with two queries against two keys, over the same values, and the second answer is taken off the first.

q = h Wq^T holds, head by head, [query of map 1 | query of map 2] (`key_dim` each), k = h Wk^T the same for every
key/value head, v = h Wv^T one value (`value_dim`) a key/value head; query head n reads key/value head
n // (heads / kv_heads).  Each map is softmax attention of its own under the causal mask (and a sliding `window`:
position i sees j with 0 <= i - j < window; 0: every earlier position) with score = q . k * scale.  With the maps'
results a1 and a2:

    o = a1 - lambda a2,    lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff      (one number a layer),
    o <- o / sqrt(mean(o^2) + eps) * (1 - diff)                                  (over a head's values, no weight),

then the output projection of the heads side by side.  `rotary` (as `sink_window_attention` takes it) rotates the
first `dims` entries of every map of every query and key head.

How it runs.  The two maps are attention with 2 heads query heads and 2 kv_heads key heads of `key_dim` that share
kv_heads value heads: the paged cache keeps a position's keys as one row [map 1 | map 2] a key/value head beside its
value, and `sink_attention` reads the half it needs (`maps=2`).  The rows of Wq are put in the order (key/value head,
map, query head of the group) when the weights are bound, so that the query heads of one key head lie side by side as
that kernel wants them.  The maps' results stay 32-bit up to the difference and its norm (`diff_combine`), whatever
the run's dtype.
"""
from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional

import torch

from .base import (MIXERS, VECTOR32, BuildEnv, KVNeed, LayerCache, Mixer, StepContext, TensorSpec, product_weight,
                   project)
from .rope import rotary_frequencies, rotary_magnitude
from .sink_attention import split_scratch


@MIXERS.register("differential_attention")
class DifferentialAttention(Mixer):
    graph_safe = True
    takes_out = True
    MAPS = 2

    def __init__(self, width: int, heads: int, kv_heads: int, key_dim: int, value_dim: int, scale: float, diff: float,
                 eps: float, prefix: str, window: int = 0, rotary: Optional[Mapping] = None,
                 names: Optional[Mapping[str, str]] = None) -> None:
        if heads % kv_heads != 0:
            raise ValueError(f"{heads} heads cannot share {kv_heads} kv heads evenly")
        if window < 0:
            raise ValueError("the window must not be negative")
        self.width, self.heads, self.kv_heads = int(width), int(heads), int(kv_heads)
        self.key_dim, self.value_dim = int(key_dim), int(value_dim)
        self.scale, self.diff, self.eps, self.window = float(scale), float(diff), float(eps), int(window)
        self.rot_dims, self.rot_interleaved, self.rot_magnitude, self.freq_table = 0, False, 1.0, []
        if rotary is not None:
            self.rot_dims = int(rotary["dims"])
            pairing = rotary.get("pairing", "half")
            if pairing not in ("half", "interleaved"):
                raise ValueError(f"rotary pairing {pairing!r} is not known (known: 'half', 'interleaved')")
            if self.rot_dims % 2 or not 2 <= self.rot_dims <= self.key_dim:
                raise ValueError(f"{self.rot_dims} rotated entries do not fit a map of {key_dim}")
            scaling = dict(rotary["scaling"]) if rotary.get("scaling") else None
            self.rot_interleaved = pairing == "interleaved"
            self.freq_table = rotary_frequencies(self.rot_dims, float(rotary["base"]), scaling)
            self.rot_magnitude = rotary_magnitude(scaling)
        n = {"q": "q", "k": "k", "v": "v", "o": "o", "lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2"}
        n.update(names or {})
        self.names: Dict[str, str] = {key: f"{prefix}.{val}" for key, val in n.items()}
        self.q_width = self.heads * self.MAPS * self.key_dim
        self.k_width = self.kv_heads * self.MAPS * self.key_dim
        self.v_width = self.kv_heads * self.value_dim
        self.o_width = self.heads * self.value_dim
        self.lam = 0.0
        self.w_in = self.w_o = self.freqs = None

    def tensor_specs(self) -> List[TensorSpec]:
        nm = self.names
        return [TensorSpec(nm["q"], (self.q_width, self.width)), TensorSpec(nm["k"], (self.k_width, self.width)),
                TensorSpec(nm["v"], (self.v_width, self.width)),
                *(TensorSpec(nm[key], (self.key_dim,), kind=VECTOR32) for key in ("lq1", "lk1", "lq2", "lk2")),
                TensorSpec(nm["o"], (self.width, self.o_width))]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        nm = self.names
        q, k, v = (tensors[nm[key]] for key in ("q", "k", "v"))
        if len({m.dtype for m in (q, k, v)}) != 1:
            raise ValueError(f"{nm['q']}: the projections of one input are stored in different dtypes")
        # Wq's rows from (head, map) to (kv head, map, head of the group): the query heads of a key head side by side
        group = self.heads // self.kv_heads
        q = q.reshape(self.kv_heads, group, self.MAPS, self.key_dim, self.width).permute(0, 2, 1, 3, 4) \
            .reshape(self.q_width, self.width)
        self.w_in = product_weight(env, torch.cat([q, k, v], dim=0))
        self.w_o = product_weight(env, tensors[nm["o"]])
        lq1, lk1, lq2, lk2 = (tensors[nm[key]].detach().to("cpu", torch.float32) for key in ("lq1", "lk1", "lq2", "lk2"))
        # one number a layer, made once in 32-bit
        self.lam = float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum()) + torch.tensor(self.diff))
        if not math.isfinite(self.lam):
            raise ValueError(f"{nm['lq1']}: the layer's lambda is not finite")
        self.freqs = torch.tensor(self.freq_table, dtype=torch.float64, device=env.device) if self.rot_dims else None

    def cache_need(self) -> KVNeed:
        # a position's keys of both maps are one row a key/value head
        return KVNeed(self.kv_heads, self.MAPS * self.key_dim, self.window, self.value_dim, 0)

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: Optional[LayerCache],
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
        if cache is None or cache.k is None:
            raise RuntimeError("attention needs a key/value cache")
        kn, rows, M = ctx.kernels, h.shape[0], self.MAPS
        total = self.q_width + self.k_width + self.v_width
        proj = ctx.ws.alloc((rows, (total + 3) // 4 * 4), torch.float32)[:, :total]
        project(kn, ctx, h, self.w_in, proj)
        q = ctx.ws.alloc((rows, self.q_width), ctx.dtype)
        k = ctx.ws.alloc((rows, self.k_width), ctx.dtype)
        v = ctx.ws.alloc((rows, self.v_width), ctx.dtype)
        # every map of every head is a head of key_dim to the rotation; the values pass
        kn.rotary_qkv(proj, q, k, v, M * self.heads, M * self.kv_heads, self.key_dim, self.value_dim, self.rot_dims,
                      self.rot_interleaved, self.freqs, self.rot_magnitude, None, ctx.row_pos, value_width=self.v_width)
        if cache.write:
            kn.kv_store(k, v, self.kv_heads, M * self.key_dim, self.value_dim, ctx.row_pos, ctx.row_seq, ctx.seq_slot,
                        cache.block_table, cache.k, cache.v, cache.block_size)
        both = ctx.ws.alloc((rows, M * self.o_width), torch.float32)
        kn.sink_attention(q, both, M * self.heads, M * self.kv_heads, self.key_dim, self.value_dim, ctx.row_pos,
                          ctx.row_seq, ctx.seq_slot, cache.block_table, cache.k, cache.v, cache.block_size, self.scale,
                          window=self.window, keep_first=0, sink=False, gate=None, decode=ctx.decode, maps=M,
                          **split_scratch(ctx, q.dtype, M * self.heads, M * self.kv_heads, self.key_dim,
                                          self.value_dim, cache.block_size, self.window, 0))
        att = ctx.ws.alloc((rows, self.o_width), ctx.dtype)
        kn.diff_combine(both, att, self.heads, self.kv_heads, self.value_dim, self.lam, self.eps, 1.0 - self.diff)
        if out is None:
            out = ctx.ws.alloc((rows, self.width), torch.float32)
        project(kn, ctx, att, self.w_o, out)
        return out
