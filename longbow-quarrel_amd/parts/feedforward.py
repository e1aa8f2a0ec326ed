"""Dense SwiGLU feed-forward: down(silu(gate(n)) * up(n)), no biases, no clamps
(internal/device/metal.go:1464-1471; silu(g) = g / (1 + e^-g),
internal/device/cpu_ref.go:132-149).  gate and up are concatenated at bind time
so that one matrix product makes both."""
from __future__ import annotations

from typing import Dict, List, Mapping, Optional

import torch

from .base import (FEED_FORWARDS, VECTOR32, BuildEnv, FeedForward, NormedRows, StepContext, TensorSpec, product_weight, project,
                   project_into, project_normed)


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True

    def __init__(self, width: int, inner: int, prefix: str, names: Optional[Mapping[str, str]] = None) -> None:
        self.width, self.inner = int(width), int(inner)
        n = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}
        n.update(names or {})
        self.names: Dict[str, str] = {key: f"{prefix}.{val}" for key, val in n.items()}
        self.fused = False
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [
            TensorSpec(self.names["gate"], (self.inner, self.width)),
            TensorSpec(self.names["up"], (self.inner, self.width)),
            TensorSpec(self.names["down"], (self.width, self.inner)),
        ]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        gate, up = tensors[self.names["gate"]], tensors[self.names["up"]]
        if gate.dtype != up.dtype:
            raise ValueError(f"{self.names['gate']}: gate and up projections are stored in different dtypes")
        kn = env.kernels
        self.fused = gate.dtype == env.dtype and self.inner % 8 == 0 and \
            getattr(kn, "linear_swiglu_supported", lambda *a: False)(gate.dtype, 2 * self.inner, self.width)
        if self.fused:
            # gate and up rows interleaved so that the product's epilogue can apply silu(g) * u itself
            self.w_gate_up = product_weight(env, kn.interleave_gate_up(gate, up))
        else:
            self.w_gate_up = product_weight(env, torch.cat([gate, up], dim=0))
        self.w_down = product_weight(env, tensors[self.names["down"]])

    takes_normed_rows = True
    takes_residual_sink = True

    def forward(self, h, ctx: StepContext, sink=None) -> Optional[torch.Tensor]:
        kn = ctx.kernels
        rows = h.shape[0]
        act = ctx.ws.alloc((rows, self.inner), ctx.dtype)
        if self.fused:
            if not project_normed(kn, ctx, h, self.w_gate_up, act, swiglu=True):
                if isinstance(h, NormedRows):
                    h = h.tensor(ctx)
                kn.linear_swiglu(h, self.w_gate_up, act)
        else:
            gu = ctx.ws.alloc((rows, 2 * self.inner), torch.float32)
            if not project_normed(kn, ctx, h, self.w_gate_up, gu):
                if isinstance(h, NormedRows):
                    h = h.tensor(ctx)
                project(kn, ctx, h, self.w_gate_up, gu)
            kn.swiglu(gu, act)
        return project_into(kn, ctx, act, self.w_down, sink)


@FEED_FORWARDS.register("glu")
class GatedLinearUnit(FeedForward):
    """down(act(gate(h)) * up(h)) with a choice of `activation` ("relu", "silu", "gelu_tanh").  gate and up are one
    matrix product whose 32-bit result the activation kernel reads.  With `bias` every projection has one
    (`<name>.b`): the activation kernel adds gate's and up's; down's is one more column of its weight, which meets a
    column of ones that the activation kernel leaves behind its result."""

    graph_safe = True
    ACTIVATIONS = ("silu", "relu", "gelu_tanh")
    BIAS_TAIL = 8  # columns behind the activations: a one and zeros (a product's K stays a multiple of eight)

    def __init__(self, width: int, inner: int, prefix: str, activation: str = "silu", bias: bool = False,
                 names: Optional[Mapping[str, str]] = None) -> None:
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {', '.join(self.ACTIVATIONS)}")
        self.width, self.inner, self.activation, self.bias = int(width), int(inner), activation, bool(bias)
        n = {"gate": "gate", "up": "up", "down": "down"}
        n.update(names or {})
        self.names: Dict[str, str] = {key: f"{prefix}.{val}" for key, val in n.items()}
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None
        self.b_gate_up: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [
            TensorSpec(self.names["gate"], (self.inner, self.width)),
            TensorSpec(self.names["up"], (self.inner, self.width)),
            TensorSpec(self.names["down"], (self.width, self.inner)),
        ]
        if self.bias:
            specs += [TensorSpec(self.names["gate"] + ".b", (self.inner,), kind=VECTOR32),
                      TensorSpec(self.names["up"] + ".b", (self.inner,), kind=VECTOR32),
                      TensorSpec(self.names["down"] + ".b", (self.width,))]  # (in the dtype of the matrix it joins)
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        gate, up = tensors[self.names["gate"]], tensors[self.names["up"]]
        if gate.dtype != up.dtype:
            raise ValueError(f"{self.names['gate']}: gate and up projections are stored in different dtypes")
        self.w_gate_up = product_weight(env, torch.cat([gate, up], dim=0))
        down = tensors[self.names["down"]]
        if self.bias:
            self.b_gate_up = torch.cat([tensors[self.names["gate"] + ".b"], tensors[self.names["up"] + ".b"]]).contiguous()
            b = tensors[self.names["down"] + ".b"].to(down.dtype)
            down = torch.cat([down, b[:, None], down.new_zeros((self.width, self.BIAS_TAIL - 1))], dim=1)
        self.w_down = product_weight(env, down)

    takes_out = True

    def forward(self, h, ctx: StepContext, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        kn = ctx.kernels
        rows = h.shape[0]
        gu = ctx.ws.alloc((rows, 2 * self.inner), torch.float32)
        project(kn, ctx, h, self.w_gate_up, gu)
        if self.bias:
            act = ctx.ws.alloc((rows, self.inner + self.BIAS_TAIL), self.w_down.dtype)
            kn.glu(gu, act, self.activation, bias=self.b_gate_up, tail=self.BIAS_TAIL)
        else:
            act = ctx.ws.alloc((rows, self.inner), ctx.dtype)
            kn.glu(gu, act, self.activation)
        if out is None:
            out = ctx.ws.alloc((rows, self.width), torch.float32)
        project(kn, ctx, act, self.w_down, out)
        return out


@FEED_FORWARDS.register("mlp")
class PlainFeedForward(FeedForward):
    """down(act(up(h))): two matrices, no gate and no biases; `activation` "gelu" (the exact one, with the error
    function), "gelu_tanh", "silu" or "relu".  The activation reads the first product's 32-bit result."""

    graph_safe = True
    takes_out = True
    ACTIVATIONS = ("gelu", "gelu_tanh", "silu", "relu")

    def __init__(self, width: int, inner: int, prefix: str, activation: str = "gelu",
                 names: Optional[Mapping[str, str]] = None) -> None:
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {', '.join(self.ACTIVATIONS)}")
        self.width, self.inner, self.activation = int(width), int(inner), activation
        n = {"up": "up", "down": "down"}
        n.update(names or {})
        self.names: Dict[str, str] = {key: f"{prefix}.{val}" for key, val in n.items()}
        self.w_up = self.w_down = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.names["up"], (self.inner, self.width)),
                TensorSpec(self.names["down"], (self.width, self.inner))]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        self.w_up = product_weight(env, tensors[self.names["up"]])
        self.w_down = product_weight(env, tensors[self.names["down"]])

    def forward(self, h, ctx: StepContext, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        kn, rows = ctx.kernels, h.shape[0]
        u = ctx.ws.alloc((rows, (self.inner + 3) // 4 * 4), torch.float32)[:, : self.inner]
        project(kn, ctx, h, self.w_up, u)
        act = ctx.ws.alloc((rows, self.inner), ctx.dtype)
        kn.activation(u, act, self.activation)
        if out is None:
            out = ctx.ws.alloc((rows, self.width), torch.float32)
        project(kn, ctx, act, self.w_down, out)
        return out


@FEED_FORWARDS.register("moe")
class MixtureOfExperts(FeedForward):
    """`experts` small gated feed-forwards of which every token uses `top`, chosen by a router.

    Router: z = Wr h summed in 32-bit (h as the run holds it), s = sigmoid(z) in 32-bit; the `top` largest scores win (the lower index on a tie); an expert's
    weight is its score as it is (`renormalize` divides the chosen scores by their sum).  With `weight_input` the
    weight multiplies what the expert reads, out = sum_e expert_e(s_e h); otherwise its result.

    Expert (`activation` "clamped_swish"): g = min(Wg h, limit), u = clamp(Wu h, -limit, limit),
    y = g sigmoid(1.702 g) (u + 1), result Wd y; no biases.  Wg (s h) = s (Wg h), so the weight is applied to the
    32-bit results of the gate and up products, ahead of the clamps.  `activation` "silu": y = silu(Wg h) (Wu h),
    no clamps.

    `correction`: a learned constant for every expert (`<prefix>.correction`) is added to the scores for the choice
    alone; the weights stay the scores.  `groups` / `keep`: the experts form `groups` equal groups of neighbours, a
    group's mark is the sum of its two largest choice scores, and only experts of the `keep` best groups can be
    chosen.  `shared_inner`: one more expert of that inner size (`<prefix>.shared.*`, the same form) runs for every
    token with weight one, and is added.  `shared_gate`: the shared expert's result is multiplied by the sigmoid of
    one more projection of the input, a number a token (`<prefix>.shared.sg`, [1, width]).

    `scoring` "softmax": s = softmax(z) over all the router's outputs in the place of the sigmoid.  `group_mark`
    "max": a group's mark is its largest choice score (the default, "top2", is the sum of its two largest); experts
    outside the kept groups cannot be chosen whatever their choice scores (which may be negative).  `renormalize_eps`
    is added to the chosen scores' sum before the division.  `identity`: so many more outputs of the router, behind
    the experts', stand for experts without tensors that hand their input on (times the weight); they take part in
    the scores, the groups and the choice like the others.

    How it runs.  The experts' gate and up matrices are one matrix [experts * 2 ff, width] and their down matrices
    one [width, experts * ff]: with the activations of the experts that a token did not choose set to zero, the down
    product adds the chosen experts' results by itself.  A step of few rows (decoding) runs every row through all
    experts' columns: a batch of more than a few tokens reads nearly all experts anyway.  A prompt step of
    `sort_from_rows` rows or more is sorted by expert first (`moe_sort`: the chosen (row, expert) couples expert by
    expert, rows ascending), the rows gathered in that order, and every expert's two products run over its own rows
    only; the results go back to their rows and are added in the order of the experts.  The host reads the experts'
    row counts for that (one wait a layer), which a captured step never does: it takes the first way."""

    graph_safe = True
    takes_out = True
    #: rows from which a step that is no decoding step is sorted by expert
    sort_from_rows = 256

    ACTIVATIONS = ("clamped_swish", "silu")

    def __init__(self, width: int, experts: int, top: int, inner: int, prefix: str, limit: float = 0.0,
                 weight_input: bool = True, renormalize: bool = False, activation: str = "clamped_swish",
                 correction: bool = False, groups: int = 0, keep: int = 0, shared_inner: int = 0,
                 names: Optional[Mapping[str, str]] = None, scoring: str = "sigmoid", group_mark: str = "top2",
                 renormalize_eps: float = 0.0, identity: int = 0, shared_gate: bool = False) -> None:
        self.width, self.experts, self.top, self.inner = int(width), int(experts), int(top), int(inner)
        self.scoring, self.group_mark, self.renormalize_eps = scoring, group_mark, float(renormalize_eps)
        self.identity, self.shared_gate = int(identity), bool(shared_gate)
        self.outputs = self.experts + self.identity  # what the router scores
        if scoring not in ("sigmoid", "softmax") or group_mark not in ("top2", "max"):
            raise ValueError(f"scoring is 'sigmoid' or 'softmax' ({scoring!r}), a group's mark 'top2' or 'max' ({group_mark!r})")
        if self.identity < 0 or (self.identity and weight_input):
            raise ValueError("identity experts: none or more, and the weight on the experts' results")
        if self.shared_gate and not shared_inner:
            raise ValueError("a gate on the shared expert needs a shared expert")
        self.limit, self.weight_input, self.renormalize = float(limit), bool(weight_input), bool(renormalize)
        self.activation, self.correction = activation, bool(correction)
        self.groups, self.keep, self.shared_inner = int(groups), int(keep), int(shared_inner)
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {', '.join(self.ACTIVATIONS)}")
        if self.shared_inner and activation != "silu":
            raise ValueError("a shared expert is built for the 'silu' activation only")
        if not 1 <= self.top <= self.outputs:
            raise ValueError(f"{top} of {self.outputs} experts cannot be chosen")
        if self.groups > 1:
            if self.outputs % self.groups or not 1 <= self.keep <= self.groups or self.groups > 64:
                raise ValueError(f"{self.outputs} experts do not form {groups} equal groups of which {keep} are kept")
            if self.keep * (self.outputs // self.groups) < self.top:
                raise ValueError(f"{keep} groups of {self.outputs // self.groups} experts cannot give {top} experts")
        else:
            self.groups = self.keep = 0
        n = {"router": "router", "expert": "e{}", "gate": "gate", "up": "up", "down": "down",
             "correction": "correction", "shared": "shared", "shared_gate": "sg"}
        n.update(names or {})
        self.prefix, self.n = prefix, n
        self.w_correction: Optional[torch.Tensor] = None

    def _name(self, e: int, what: str) -> str:
        return f"{self.prefix}.{self.n['expert'].format(e)}.{self.n[what]}"

    def _shared_name(self, what: str) -> str:
        return f"{self.prefix}.{self.n['shared']}.{self.n[what]}"

    def tensor_specs(self) -> List[TensorSpec]:
        specs = []
        for e in range(self.experts):
            specs += [TensorSpec(self._name(e, "gate"), (self.inner, self.width)),
                      TensorSpec(self._name(e, "up"), (self.inner, self.width)),
                      TensorSpec(self._name(e, "down"), (self.width, self.inner))]
        specs.append(TensorSpec(f"{self.prefix}.{self.n['router']}", (self.outputs, self.width)))
        if self.correction:
            specs.append(TensorSpec(f"{self.prefix}.{self.n['correction']}", (self.outputs,), kind=VECTOR32))
        if self.shared_inner:
            specs += [TensorSpec(self._shared_name("gate"), (self.shared_inner, self.width)),
                      TensorSpec(self._shared_name("up"), (self.shared_inner, self.width)),
                      TensorSpec(self._shared_name("down"), (self.width, self.shared_inner))]
        if self.shared_gate:
            specs.append(TensorSpec(self._shared_name("shared_gate"), (1, self.width)))
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        E = self.experts
        gu = [tensors[self._name(e, w)] for e in range(E) for w in ("gate", "up")]
        down = [tensors[self._name(e, "down")] for e in range(E)]
        ffs = self.shared_inner
        if ffs:  # the shared expert's rows and columns lie behind the routed experts'
            gu += [tensors[self._shared_name(w)] for w in ("gate", "up")]
            down.append(tensors[self._shared_name("down")])
        if len({m.dtype for m in gu + down}) != 1:
            raise ValueError(f"{self._name(0, 'gate')}: the experts' matrices are stored in different dtypes")
        # expert e's rows of the first matrix: [gate (ff) | up (ff)]; its columns of the second: e ff .. (e + 1) ff
        ff = self.inner
        runs = [(e * 2 * ff, 2 * ff) for e in range(E)] + ([(E * 2 * ff, 2 * ffs)] if ffs else [])
        whole = torch.cat(gu, dim=0).contiguous()  # [E * 2 ff (+ 2 ffs), width]
        self.w_gate_up = product_weight(env, whole)
        rows_of = getattr(env.kernels, "weight_rows", None)
        if self.w_gate_up is whole:
            self.gate_up_of = [whole[at : at + n] for at, n in runs]
        else:  # held in the products' own order: an expert's rows must be a weight in that order too
            self.gate_up_of = [rows_of(self.w_gate_up, at, n) if rows_of else None for at, n in runs]
            if any(w is None for w in self.gate_up_of):
                self.w_gate_up = whole
                self.gate_up_of = [whole[at : at + n] for at, n in runs]
        # the second matrix stays dense: an expert is a run of its columns, which only the dense order can give
        self.w_down = torch.cat(down, dim=1).contiguous()  # [width, E * ff (+ ffs)]
        self.down_of = [self.w_down[:, e * ff : (e + 1) * ff] for e in range(E)]
        if ffs:
            self.down_of.append(self.w_down[:, E * ff :])
        if self.correction:
            self.w_correction = tensors[f"{self.prefix}.{self.n['correction']}"].contiguous()
        # the router's product as it is stored: bfloat16 operands multiply exactly into 32-bit sums, and its result
        # (the logits) and everything after it are 32-bit
        self.w_router = tensors[f"{self.prefix}.{self.n['router']}"]
        if self.shared_gate:  # the gate's logit rides in the router's product, as one more row behind its own
            sg = tensors[self._shared_name("shared_gate")]
            if sg.dtype != self.w_router.dtype:
                raise ValueError(f"{self._shared_name('shared_gate')}: stored in another dtype than the router")
            self.w_router = torch.cat([self.w_router, sg.reshape(1, self.width)], dim=0)
        self.w_router = self.w_router.contiguous()

    def _route(self, h, ctx: StepContext) -> torch.Tensor:
        """The weight of every expert for every row (-1: not chosen).  Leaves the identity experts' weights and the
        shared expert's gate logits of this step in `self._step`."""
        kn, rows, E, N = ctx.kernels, h.shape[0], self.experts, self.outputs
        nz = N + (1 if self.shared_gate else 0)
        z = ctx.ws.alloc((rows, (nz + 3) // 4 * 4), torch.float32)[:, :nz]
        project(kn, ctx, h, self.w_router, z)
        route = ctx.ws.alloc((rows, E), torch.float32)  # the weight of a chosen expert, -1 for the others
        more = {}
        if self.correction:
            more["correction"] = self.w_correction
        if self.groups > 1:
            more.update(groups=self.groups, keep=self.keep)
        if self.scoring != "sigmoid":
            more["scoring"] = self.scoring
        if self.group_mark != "top2":
            more["group_mark"] = self.group_mark
        if self.renormalize_eps:
            more["renormalize_eps"] = self.renormalize_eps
        passed = None
        if self.identity:
            passed = more["identity"] = ctx.ws.alloc((rows, self.identity), torch.float32)
        kn.moe_route(z[:, :N], route, self.top, self.renormalize, **more)
        self._step = (passed, z[:, N:] if self.shared_gate else None)
        return route

    def _pass_on(self, h, out, ctx: StepContext) -> None:
        """The identity experts' share: out += h * (the sum of the chosen identity experts' weights)."""
        passed = self._step[0]
        if passed is not None:
            ctx.kernels.moe_identity(h, passed, out)

    def _sorts(self, rows: int, ctx: StepContext) -> bool:
        return rows >= self.sort_from_rows and not ctx.decode and not ctx.dry and self.outputs > self.top \
            and getattr(ctx.kernels, "moe_sort", None) is not None

    def _unit(self, gu, act, ctx: StepContext) -> None:
        """The shared expert's activation (no routing; weight one, or the sigmoid of its gate's logit)."""
        gate = self._step[1]
        if gate is not None:
            ctx.kernels.glu(gu, act, "silu", row_gate=gate)
        else:
            ctx.kernels.glu(gu, act, "silu")

    def forward_pieces(self, h, ctx: StepContext):
        """The result in pieces [n, rows, width] that the caller adds: the routed experts' sum, and the shared
        expert's result where a step's rows were sorted by expert (otherwise one product adds both)."""
        rows = h.shape[0]
        if not (self.shared_inner and self._sorts(rows, ctx)):
            out = ctx.ws.alloc((1, rows, self.width), torch.float32)
            self.forward(h, ctx, out=out[0])
            return out, (1.0,)
        out = ctx.ws.alloc((2, rows, self.width), torch.float32)
        self._sorted(h, self._route(h, ctx), out[0], ctx)
        self._pass_on(h, out[0], ctx)
        self._shared(h, out[1], ctx)
        return out, (1.0, 1.0)

    def _shared(self, h, out, ctx: StepContext) -> None:
        kn, rows, ffs = ctx.kernels, h.shape[0], self.shared_inner
        gu = ctx.ws.alloc((rows, 2 * ffs), torch.float32)
        project(kn, ctx, h, self.gate_up_of[-1], gu)
        act = ctx.ws.alloc((rows, ffs), ctx.dtype)
        self._unit(gu, act, ctx)
        project(kn, ctx, act, self.down_of[-1], out)

    def forward(self, h, ctx: StepContext, out: Optional[torch.Tensor] = None) -> torch.Tensor:
        kn = ctx.kernels
        rows, E, ff, ffs = h.shape[0], self.experts, self.inner, self.shared_inner
        route = self._route(h, ctx)
        if out is None:
            out = ctx.ws.alloc((rows, self.width), torch.float32)
        if self._sorts(rows, ctx):
            self._sorted(h, route, out, ctx)
            self._pass_on(h, out, ctx)
            if ffs:
                extra = ctx.ws.alloc((rows, self.width), torch.float32)
                self._shared(h, extra, ctx)
                kn.add(out, extra)
            return out
        # every row through all experts' columns (and the shared expert's behind them): the activations of the
        # experts that a row did not choose are zeros, so the second product adds the chosen ones and the shared one
        gu = ctx.ws.alloc((rows, E * 2 * ff + 2 * ffs), torch.float32)
        project(kn, ctx, h, self.w_gate_up, gu)
        act = ctx.ws.alloc((rows, E * ff + ffs), ctx.dtype)
        more = {"activation": self.activation} if self.activation != "clamped_swish" else {}
        kn.moe_glu(gu[:, : E * 2 * ff], route, act[:, : E * ff], E, ff, self.limit, self.weight_input, **more)
        if ffs:
            self._unit(gu[:, E * 2 * ff :], act[:, E * ff :], ctx)
        project(kn, ctx, act, self.w_down, out)
        self._pass_on(h, out, ctx)
        return out

    def _sorted(self, h, route, out, ctx: StepContext) -> None:
        """The step's rows sorted by expert: every expert's products over its own rows only."""
        kn = ctx.kernels
        rows, E, ff, top = h.shape[0], self.experts, self.inner, self.top
        pairs = rows * top
        counts = ctx.ws.alloc((E,), torch.int32)
        order = ctx.ws.alloc((pairs,), torch.int32)       # sorted place -> row
        weight = ctx.ws.alloc((pairs, 1), torch.float32)  # sorted place -> the row's weight for its expert
        place_of = ctx.ws.alloc((rows, E), torch.int32)   # (row, expert) -> sorted place, or -1
        kn.moe_sort(route, counts, order, weight, place_of)
        n_of = counts.tolist()  # the one wait: the products below are launched with every expert's number of rows
        total = sum(n_of)
        if total == 0:
            kn.moe_scatter(out, place_of, out)  # (no row chose anything: zeros)
            return
        hs = ctx.ws.alloc((pairs, self.width), h.dtype)
        kn.moe_gather(h, order, hs, total)
        gu = ctx.ws.alloc((pairs, 2 * ff), torch.float32)
        at = 0
        for e, n in enumerate(n_of):
            if n:
                project(kn, ctx, hs[at : at + n], self.gate_up_of[e], gu[at : at + n])
                at += n
        act = ctx.ws.alloc((pairs, ff), ctx.dtype)
        more = {"activation": self.activation} if self.activation != "clamped_swish" else {}
        kn.moe_glu(gu[:total], weight[:total], act[:total], 1, ff, self.limit, self.weight_input, **more)
        ys = ctx.ws.alloc((pairs, self.width), torch.float32)
        at = 0
        for e, n in enumerate(n_of):
            if n:
                project(kn, ctx, act[at : at + n], self.down_of[e], ys[at : at + n])
                at += n
        kn.moe_scatter(ys, place_of, out)
