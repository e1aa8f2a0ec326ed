"""Mixers with a recurrent state of fixed size per sequence: the Mamba-2 state-space layer and the gated
delta rule.  Both carry, for every sequence, a matrix state per head in 32-bit and the last inputs of a
short causal convolution; both are computed token by token in the order of the sequence, by one kernel for
prompts and single tokens alike, so that the result does not depend on how a sequence is cut into steps.

Everything that enters a recurrence is 32-bit (step sizes, decays, gates, unit norms, the state); the
projections are products in the run's dtype with 32-bit results.
"""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional

import torch

from .base import (MIXERS, VECTOR32, BuildEnv, Mixer, MultiCache, MultiNeed, StateNeed, StepContext, TensorSpec,
                   product_weight, project)


def _round4(n: int) -> int:
    return (n + 3) // 4 * 4


class _Recurrent(Mixer):
    graph_safe = True
    takes_out = True

    @staticmethod
    def _states(cache):
        if not isinstance(cache, MultiCache) or len(cache.parts) != 2:
            raise RuntimeError("a recurrent mixer needs its state and its convolution's last inputs")
        if not cache.write:
            raise RuntimeError("a recurrent state cannot be shared between runs of the schedule")
        return cache.parts[0].state, cache.parts[1].state


@MIXERS.register("mamba2")
class Mamba2(_Recurrent):
    """The state-space layer of Dao and Gu, "Transformers are SSMs: Generalized Models and Efficient Algorithms
    Through Structured State Space Duality".  One product of the input gives [z | x | B | C | dt] (inner =
    heads * head_dim columns for z and x, groups * state for B and C, heads for dt).  x, B and C pass a causal
    convolution per channel (`conv` taps, with bias) and silu.  dt = softplus(dt + dt_bias).  Per head h (its B
    and C are those of group h // (heads / groups)), with the state S [state, head_dim] starting at zero:

        S <- exp(-exp(A_log_h) dt) S + dt B x^T,      y = S^T C + D_h x.

    Then y silu(z), an RMS norm in `norm_groups` equal parts (each by its own root mean square) times a
    weight, and the output projection."""

    def __init__(self, width: int, heads: int, head_dim: int, state: int, groups: int, conv: int, norm_groups: int,
                 eps: float, prefix: str, names: Optional[Mapping[str, str]] = None) -> None:
        if heads % groups != 0:
            raise ValueError(f"{heads} heads cannot share {groups} groups evenly")
        self.width, self.heads, self.head_dim = int(width), int(heads), int(head_dim)
        self.state, self.groups, self.taps = int(state), int(groups), int(conv)
        self.norm_groups, self.eps = int(norm_groups), float(eps)
        self.inner = self.heads * self.head_dim
        if self.norm_groups <= 0 or self.inner % self.norm_groups != 0:
            raise ValueError(f"{self.inner} channels cannot be normed in {norm_groups} equal parts")
        if self.taps < 1:
            raise ValueError("the convolution needs at least one tap")
        self.conv_channels = self.inner + 2 * self.groups * self.state
        self.in_width = 2 * self.inner + 2 * self.groups * self.state + self.heads
        n = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "dt_bias": "dt_bias", "A_log": "A_log", "D": "D",
             "norm": "norm", "o": "o"}
        n.update(names or {})
        self.names: Dict[str, str] = {key: f"{prefix}.{val}" for key, val in n.items()}

    def tensor_specs(self) -> List[TensorSpec]:
        nm = self.names
        return [
            TensorSpec(nm["in"], (self.in_width, self.width)),
            TensorSpec(nm["conv"], (self.conv_channels, self.taps), kind=VECTOR32),
            TensorSpec(nm["conv_bias"], (self.conv_channels,), kind=VECTOR32),
            TensorSpec(nm["dt_bias"], (self.heads,), kind=VECTOR32),
            TensorSpec(nm["A_log"], (self.heads,), kind=VECTOR32),
            TensorSpec(nm["D"], (self.heads,), kind=VECTOR32, init="around_one"),
            TensorSpec(nm["norm"], (self.inner,), kind=VECTOR32, init="around_one"),
            TensorSpec(nm["o"], (self.width, self.inner)),
        ]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        nm = self.names
        self.w_in = product_weight(env, tensors[nm["in"]])
        self.w_o = product_weight(env, tensors[nm["o"]])
        self.conv_w = tensors[nm["conv"]].contiguous()
        self.conv_b = tensors[nm["conv_bias"]].contiguous()
        self.dt_bias, self.a_log, self.d, self.norm_w = (tensors[nm[k]].contiguous() for k in
                                                         ("dt_bias", "A_log", "D", "norm"))

    def cache_need(self) -> MultiNeed:
        # the state is held [head, head_dim, state]: a thread of the scan owns a run of one column
        return MultiNeed((StateNeed((self.heads, self.head_dim, self.state), torch.float32),
                          StateNeed((max(1, self.taps - 1), self.conv_channels), torch.float32)))

    def forward(self, h: torch.Tensor, ctx: StepContext, cache, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        kn = ctx.kernels
        state, conv_state = self._states(cache)
        rows = h.shape[0]
        gn = self.groups * self.state
        u = ctx.ws.alloc((rows, _round4(self.in_width)), torch.float32)[:, : self.in_width]
        project(kn, ctx, h, self.w_in, u)
        z = u[:, : self.inner]
        dt = u[:, 2 * self.inner + 2 * gn :]
        xbc = ctx.ws.alloc((rows, _round4(self.conv_channels)), torch.float32)[:, : self.conv_channels]
        kn.causal_conv(u[:, self.inner : self.inner + self.conv_channels], self.conv_w, self.conv_b, conv_state, xbc,
                       ctx.row_pos, ctx.row_seq, ctx.seq_slot, ctx.seq_start, ctx.seq_len, ctx.cu_rows, ctx.batch,
                       activation="silu")
        y = ctx.ws.alloc((rows, self.inner), torch.float32)
        # a few long prompts: the kernel may cut them into segments that run side by side, given scratch
        ask = getattr(kn, "ssd_scan_workspace", None)
        need = ask(ctx.batch, self.heads, self.head_dim, self.state, ctx.max_new) if ask is not None else 0
        more = dict(max_rows=ctx.max_new, workspace=ctx.ws.alloc((need,), torch.float32)) if need else {}
        kn.ssd_scan(xbc[:, : self.inner], xbc[:, self.inner : self.inner + gn], xbc[:, self.inner + gn :], dt,
                    self.dt_bias, self.a_log, self.d, state, y, self.heads, self.head_dim, self.state, self.groups,
                    ctx.seq_slot, ctx.cu_rows, ctx.batch, **more)
        normed = ctx.ws.alloc((rows, self.inner), ctx.dtype)
        kn.gated_rmsnorm(y, z, self.norm_w, self.eps, self.inner // self.norm_groups, normed, gate_first=True)
        if out is None:
            out = ctx.ws.alloc((rows, self.width), torch.float32)
        project(kn, ctx, normed, self.w_o, out)
        return out


@MIXERS.register("gated_delta")
class GatedDelta(_Recurrent):
    """The gated delta rule (Yang, Kautz, Hatamizadeh: "Gated Delta Networks: Improving Mamba2 with Delta
    Rule").  q and k are `kv_heads` x `key_dim`, v is `heads` x `value_dim`; head h uses q/k head
    h // (heads / kv_heads).  Each of q, k, v passes a short causal convolution per channel (no bias) and
    silu; q and k become unit vectors per head (x / sqrt(sum x^2 + 1e-6)) and q is scaled by key_dim^(-1/2).
    beta = sigmoid(h Wb^T) and the decay g = exp(-exp(A_log) softplus(h Wa^T + dt_bias)) are one number a head.
    Per head, with the state S [key_dim, value_dim] starting at zero:

        S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q.

    Each head's o is divided by its root mean square, multiplied by a weight that the heads share and by
    silu of one more projection of the input; then the output projection.

    `decay="channel"`: one decay for every key channel of every head, g = exp(-exp(A_log_h) softplus(W2 (W1 h) +
    dt_bias)) with dt_bias [heads * key_dim] and the two matrices a bottleneck of `decay_rank` columns; S <- diag(g) S
    multiplies the state's rows of a key channel.  `gate="sigmoid"`: the sigmoid of the gate's projection in the
    place of silu; `gate_rank`: that projection through a bottleneck of so many columns (two matrices)."""

    UNIT_EPS = 1e-6

    def __init__(self, width: int, heads: int, kv_heads: int, key_dim: int, value_dim: int, conv: int, eps: float,
                 prefix: str, decay: str = "head", decay_rank: Optional[int] = None, gate: str = "silu",
                 gate_rank: Optional[int] = None, names: Optional[Mapping[str, str]] = None) -> None:
        if heads % kv_heads != 0:
            raise ValueError(f"{heads} heads cannot share {kv_heads} q/k heads evenly")
        if decay not in ("head", "channel") or gate not in ("silu", "sigmoid"):
            raise ValueError(f"the decay is 'head' or 'channel' (found {decay!r}), the gate 'silu' or 'sigmoid' ({gate!r})")
        if decay == "channel" and (decay_rank is None or int(decay_rank) < 1):
            raise ValueError("a decay for every key channel comes through a bottleneck: its rank is needed")
        if gate_rank is not None and int(gate_rank) < 1:
            raise ValueError("the gate's bottleneck needs a rank of at least one")
        self.width, self.heads, self.kv_heads = int(width), int(heads), int(kv_heads)
        self.key_dim, self.value_dim, self.taps, self.eps = int(key_dim), int(value_dim), int(conv), float(eps)
        if self.taps < 1:
            raise ValueError("the convolution needs at least one tap")
        self.channel_decay, self.gate_act = decay == "channel", gate
        self.decay_rank = int(decay_rank) if self.channel_decay else 0
        self.gate_rank = int(gate_rank) if gate_rank is not None else 0
        self.qk_width = self.kv_heads * self.key_dim
        self.v_width = self.heads * self.value_dim
        self.conv_channels = 2 * self.qk_width + self.v_width
        self.n_decay = self.heads * self.key_dim if self.channel_decay else self.heads
        n = {"q": "q", "k": "k", "v": "v", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "beta": "b",
             "a": "a", "a1": "a1", "a2": "a2", "A_log": "A_log", "dt_bias": "dt_bias", "norm": "norm", "gate": "g",
             "g1": "g1", "g2": "g2", "o": "o"}
        n.update(names or {})
        self.names: Dict[str, str] = {key: f"{prefix}.{val}" for key, val in n.items()}

    def tensor_specs(self) -> List[TensorSpec]:
        nm = self.names
        return [
            TensorSpec(nm["q"], (self.qk_width, self.width)),
            TensorSpec(nm["q_conv"], (self.qk_width, self.taps), kind=VECTOR32),
            TensorSpec(nm["k"], (self.qk_width, self.width)),
            TensorSpec(nm["k_conv"], (self.qk_width, self.taps), kind=VECTOR32),
            TensorSpec(nm["v"], (self.v_width, self.width)),
            TensorSpec(nm["v_conv"], (self.v_width, self.taps), kind=VECTOR32),
            TensorSpec(nm["beta"], (self.heads, self.width)),
            TensorSpec(nm["A_log"], (self.heads,), kind=VECTOR32),
            TensorSpec(nm["norm"], (self.value_dim,), kind=VECTOR32, init="around_one"),
            *([TensorSpec(nm["a1"], (self.decay_rank, self.width)), TensorSpec(nm["a2"], (self.n_decay, self.decay_rank))]
              if self.channel_decay else [TensorSpec(nm["a"], (self.heads, self.width))]),
            TensorSpec(nm["dt_bias"], (self.n_decay,), kind=VECTOR32),
            *([TensorSpec(nm["g1"], (self.gate_rank, self.width)), TensorSpec(nm["g2"], (self.v_width, self.gate_rank))]
              if self.gate_rank else [TensorSpec(nm["gate"], (self.v_width, self.width))]),
            TensorSpec(nm["o"], (self.width, self.v_width)),
        ]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        nm = self.names
        # one product of the input for everything that is read in 32-bit: [q | k | v | beta (| a) (| gate)]
        whole = ["q", "k", "v", "beta"] + ([] if self.channel_decay else ["a"]) + ([] if self.gate_rank else ["gate"])
        low = (["a1"] if self.channel_decay else []) + (["g1"] if self.gate_rank else [])
        mats = [tensors[nm[k]] for k in whole + low]
        if len({m.dtype for m in mats}) != 1:
            raise ValueError(f"{nm['q']}: the projections of one input are stored in different dtypes")
        self.w_in = product_weight(env, torch.cat(mats[: len(whole)], dim=0))
        # the bottlenecks' first matrices are one product of their own: its result feeds the second matrices in the
        # run's dtype; each bottleneck's columns start on a multiple of eight
        self.w_low, self.low_at, at = None, {}, 0
        if low:
            padded = []
            for key in low:
                m = tensors[nm[key]]
                self.low_at[key] = at
                pad = (-m.shape[0]) % 8
                padded += [m] + ([m.new_zeros((pad, m.shape[1]))] if pad else [])
                at += m.shape[0] + pad
            self.w_low = product_weight(env, torch.cat(padded, dim=0))
        self.low_width = at
        self.w_a2 = product_weight(env, tensors[nm["a2"]]) if self.channel_decay else None
        self.w_g2 = product_weight(env, tensors[nm["g2"]]) if self.gate_rank else None
        self.w_o = product_weight(env, tensors[nm["o"]])
        self.conv_w = torch.cat([tensors[nm[k]] for k in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.a_log, self.dt_bias, self.norm_w = (tensors[nm[k]].contiguous() for k in ("A_log", "dt_bias", "norm"))

    def cache_need(self) -> MultiNeed:
        return MultiNeed((StateNeed((self.heads, self.value_dim, self.key_dim), torch.float32),
                          StateNeed((max(1, self.taps - 1), self.conv_channels), torch.float32)))

    def forward(self, h: torch.Tensor, ctx: StepContext, cache, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        kn = ctx.kernels
        state, conv_state = self._states(cache)
        rows = h.shape[0]
        cc, nh = self.conv_channels, self.heads
        n_a = 0 if self.channel_decay else nh
        total = cc + nh + n_a + (0 if self.gate_rank else self.v_width)
        u = ctx.ws.alloc((rows, _round4(total)), torch.float32)[:, :total]
        project(kn, ctx, h, self.w_in, u)
        decay, gate = u[:, cc + nh : cc + nh + n_a], u[:, cc + nh + n_a :]
        if self.w_low is not None:
            low = ctx.ws.alloc((rows, self.low_width), self.w_low.dtype)
            project(kn, ctx, h, self.w_low, low)
            if self.channel_decay:
                at = self.low_at["a1"]
                decay = ctx.ws.alloc((rows, self.n_decay), torch.float32)
                project(kn, ctx, low[:, at : at + self.decay_rank], self.w_a2, decay)
            if self.gate_rank:
                at = self.low_at["g1"]
                gate = ctx.ws.alloc((rows, self.v_width), torch.float32)
                project(kn, ctx, low[:, at : at + self.gate_rank], self.w_g2, gate)
        qkv = ctx.ws.alloc((rows, _round4(cc)), torch.float32)[:, :cc]
        kn.causal_conv(u[:, :cc], self.conv_w, None, conv_state, qkv, ctx.row_pos, ctx.row_seq, ctx.seq_slot,
                       ctx.seq_start, ctx.seq_len, ctx.cu_rows, ctx.batch, activation="silu")
        o = ctx.ws.alloc((rows, self.v_width), torch.float32)
        more = {"channel_decay": True} if self.channel_decay else {}
        kn.delta_scan(qkv[:, : self.qk_width], qkv[:, self.qk_width : 2 * self.qk_width], qkv[:, 2 * self.qk_width :],
                      u[:, cc : cc + nh], decay, self.dt_bias, self.a_log, state, o, self.heads,
                      self.kv_heads, self.key_dim, self.value_dim, self.key_dim ** -0.5, self.UNIT_EPS,
                      ctx.seq_slot, ctx.cu_rows, ctx.batch, **more)
        normed = ctx.ws.alloc((rows, self.v_width), ctx.dtype)
        more = {"gate": "sigmoid"} if self.gate_act == "sigmoid" else {}
        kn.gated_rmsnorm(o, gate, self.norm_w, self.eps, self.value_dim, normed, gate_first=False, **more)
        if out is None:
            out = ctx.ws.alloc((rows, self.width), torch.float32)
        project(kn, ctx, normed, self.w_o, out)
        return out


@MIXERS.register("side_by_side")
class SideBySide(Mixer):
    """Several mixers that read the same input; the result is the mean of their outputs, each first divided
    by its root mean square over the width and multiplied by a weight of its own (`out_names`).  With `weights`
    (a constant for each mixer) instead: the weighted sum of the outputs as they are, sum_i weights[i] * mixer_i(h);
    a block that takes a result in pieces gets the outputs and the constants (`forward_pieces`)."""

    takes_out = True

    def __init__(self, width: int, eps: float, sides, out_names=(), weights=None) -> None:
        self.width, self.eps = int(width), float(eps)
        self.sides = [MIXERS.get(s.kind)(**dict(s.params)) for s in sides]
        self.out_names = list(out_names)
        self.weights = None if weights is None else tuple(float(w) for w in weights)
        if not 1 <= len(self.sides) <= 4:
            raise ValueError("one to four mixers side by side")
        if self.weights is None and len(self.sides) != len(self.out_names):
            raise ValueError("mixers side by side: each with the name of its output weight, or a constant for each")
        if self.weights is not None and (len(self.weights) != len(self.sides) or self.out_names):
            raise ValueError("mixers side by side: a constant for each mixer, and then no output weights")
        self.out_w: List[torch.Tensor] = []

    @property
    def graph_safe(self) -> bool:
        return all(s.graph_safe for s in self.sides)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [s for side in self.sides for s in side.tensor_specs()]
        return specs + [TensorSpec(n, (self.width,), kind=VECTOR32, init="around_one") for n in self.out_names]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        for side in self.sides:
            side.bind(tensors, env)
        self.out_w = [tensors[n].contiguous() for n in self.out_names]

    def cache_need(self) -> MultiNeed:
        return MultiNeed(tuple(_need_or_nothing(s.cache_need()) for s in self.sides))

    def length_bound(self, kernels, longest: int) -> int:
        return max(s.length_bound(kernels, longest) for s in self.sides)

    def lengths_uneven(self, kernels, lengths) -> bool:
        return any(s.lengths_uneven(kernels, lengths) for s in self.sides)

    def _results(self, h: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        if not isinstance(cache, MultiCache) or len(cache.parts) != len(self.sides):
            raise RuntimeError("mixers side by side need a cache for each side")
        rows = h.shape[0]
        results = ctx.ws.alloc((len(self.sides), rows, self.width), torch.float32)
        for i, (side, part) in enumerate(zip(self.sides, cache.parts)):
            part = None if isinstance(part, MultiCache) and not part.parts else part
            if side.takes_out:
                side.forward(h, ctx, part, out=results[i])
            else:
                ctx.kernels.cast(side.forward(h, ctx, part), results[i])
        return results

    def forward_pieces(self, h: torch.Tensor, ctx: StepContext, cache):
        """The mixers' outputs [n, rows, width] and the constants their sum is weighted with (a weighted sum only)."""
        if self.weights is None:
            return self.forward(h, ctx, cache), (1.0,)
        return self._results(h, ctx, cache), self.weights

    def forward(self, h: torch.Tensor, ctx: StepContext, cache, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        results = self._results(h, ctx, cache)
        if out is None:
            out = ctx.ws.alloc((h.shape[0], self.width), torch.float32)
        if self.weights is None:
            ctx.kernels.rmsnorm_mean(results, self.out_w, self.eps, out)
            return out
        ctx.kernels.cast(results[0], out)
        ctx.kernels.scale(out, self.weights[0])
        for piece, weight in zip(results[1:], self.weights[1:]):
            ctx.kernels.add_scaled(out, piece, weight)
        return out


def _need_or_nothing(need):
    return need if need is not None else MultiNeed(())


@MIXERS.register("gated_linear_attention")
class GatedLinearAttention(Mixer):
    """Linear attention with a decay per key channel (Yang, Wang, Shen, Panda, Kim: "Gated Linear Attention
    Transformers with Hardware-Efficient Training").  q and k are `heads` x `key_dim`, v is `heads` x `value_dim`;
    q is scaled by key_dim^(-1/2).  The decay comes through a bottleneck of `decay_rank` columns:
    a = sigmoid(W2 (W1 h) + b)^(1 / tau), one number for every key channel of every head.  Per head, with the state
    S [key_dim, value_dim] starting at zero:

        S <- diag(a) S + k v^T,      o = S^T q.

    Each head's o is divided by its root mean square over value_dim and multiplied by a weight that the heads share,
    then by silu of one more projection of the input; then the output projection.  The decay, its logarithm and the
    state are 32-bit; one kernel walks prompts and single tokens alike, token by token."""

    graph_safe = True
    takes_out = True

    def __init__(self, width: int, heads: int, key_dim: int, value_dim: int, decay_rank: int, tau: float, eps: float,
                 prefix: str, names: Optional[Mapping[str, str]] = None) -> None:
        self.width, self.heads, self.key_dim, self.value_dim = int(width), int(heads), int(key_dim), int(value_dim)
        self.decay_rank, self.tau, self.eps = int(decay_rank), float(tau), float(eps)
        if self.tau <= 0 or self.decay_rank < 1:
            raise ValueError("the decay needs a positive tau and a rank of at least one")
        self.qk_width, self.v_width = self.heads * self.key_dim, self.heads * self.value_dim
        n = {"q": "q", "k": "k", "v": "v", "gate": "g", "a1": "a1", "a2": "a2", "a2_bias": "a2.b", "norm": "norm",
             "o": "o"}
        n.update(names or {})
        self.names: Dict[str, str] = {key: f"{prefix}.{val}" for key, val in n.items()}

    def tensor_specs(self) -> List[TensorSpec]:
        nm = self.names
        return [
            TensorSpec(nm["q"], (self.qk_width, self.width)),
            TensorSpec(nm["k"], (self.qk_width, self.width)),
            TensorSpec(nm["v"], (self.v_width, self.width)),
            TensorSpec(nm["gate"], (self.v_width, self.width)),
            TensorSpec(nm["o"], (self.width, self.v_width)),
            TensorSpec(nm["norm"], (self.value_dim,), kind=VECTOR32, init="around_one"),
            TensorSpec(nm["a1"], (self.decay_rank, self.width)),
            TensorSpec(nm["a2"], (self.qk_width, self.decay_rank)),
            TensorSpec(nm["a2_bias"], (self.qk_width,), kind=VECTOR32),
        ]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        nm = self.names
        mats = [tensors[nm[k]] for k in ("q", "k", "v", "gate")]
        if len({m.dtype for m in mats}) != 1:
            raise ValueError(f"{nm['q']}: the projections of one input are stored in different dtypes")
        self.w_in = product_weight(env, torch.cat(mats, dim=0))  # [q | k | v | gate]: 32-bit results for the scan
        # the bottleneck is a product of its own: its result feeds the next product in the run's dtype
        self.w_a1 = product_weight(env, tensors[nm["a1"]])
        self.w_a2 = product_weight(env, tensors[nm["a2"]])
        self.w_o = product_weight(env, tensors[nm["o"]])
        self.a2_bias, self.norm_w = tensors[nm["a2_bias"]].contiguous(), tensors[nm["norm"]].contiguous()

    def cache_need(self) -> StateNeed:
        # held [head, value_dim, key_dim]: a thread of the scan owns a run of one column's key channels
        return StateNeed((self.heads, self.value_dim, self.key_dim), torch.float32)

    def forward(self, h: torch.Tensor, ctx: StepContext, cache, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        kn = ctx.kernels
        if cache is None or getattr(cache, "state", None) is None:
            raise RuntimeError("gated linear attention needs its state")
        if not cache.write:
            raise RuntimeError("a recurrent state cannot be shared between runs of the schedule")
        rows = h.shape[0]
        qk, vw, rank = self.qk_width, self.v_width, self.decay_rank
        total = 2 * qk + 2 * vw
        u = ctx.ws.alloc((rows, _round4(total)), torch.float32)[:, :total]
        project(kn, ctx, h, self.w_in, u)
        low = ctx.ws.alloc((rows, (rank + 7) // 8 * 8), self.w_a2.dtype)[:, :rank]
        project(kn, ctx, h, self.w_a1, low)
        z = ctx.ws.alloc((rows, qk), torch.float32)
        project(kn, ctx, low, self.w_a2, z)
        o = ctx.ws.alloc((rows, vw), torch.float32)
        # a few long prompts: the kernel may cut them into segments that run side by side, given scratch
        ask = getattr(kn, "gla_scan_workspace", None)
        need = ask(ctx.batch, self.heads, self.key_dim, self.value_dim, ctx.max_new) if ask is not None else 0
        more = dict(max_rows=ctx.max_new, workspace=ctx.ws.alloc((need,), torch.float32)) if need else {}
        kn.gla_scan(u[:, :qk], u[:, qk : 2 * qk], u[:, 2 * qk : 2 * qk + vw], z, self.a2_bias, cache.state, o,
                    self.heads, self.key_dim, self.value_dim, self.key_dim ** -0.5, 1.0 / self.tau,
                    ctx.seq_slot, ctx.cu_rows, ctx.batch, **more)
        normed = ctx.ws.alloc((rows, vw), ctx.dtype)
        kn.gated_rmsnorm(o, u[:, 2 * qk + vw : 2 * qk + 2 * vw], self.norm_w, self.eps, self.value_dim, normed,
                         gate_first=False)
        if out is None:
            out = ctx.ws.alloc((rows, self.width), torch.float32)
        project(kn, ctx, normed, self.w_o, out)
        return out
