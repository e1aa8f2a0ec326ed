"""The pre-norm decoder block: x += mixer(norm(x)); x += ffn(norm(x))
(internal/device/metal.go:1326-1527: norm :1349, residual :1434, second norm
:1451, residual :1474).  The residual stream stays float32; each add rides on
the norm kernel that follows it, or, for the few rows of a decoding step, on the projection that
produced it, which then also leaves the statistics for the norm that the next projection folds in."""
from __future__ import annotations

import dataclasses
from typing import List, Mapping, Optional

import torch

from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, Block, BuildEnv, LayerCache, NormedRows, PartSpec,
                   ResidualSink, RowStats, StepContext, TensorSpec, build_part)


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    def __init__(self, mixer: PartSpec, feed_forward: Optional[PartSpec], mixer_norm: PartSpec,
                 ffn_norm: Optional[PartSpec]) -> None:
        """`feed_forward=None`: the layer is its mixer alone.  The norm of a feed-forward that is absent may be named
        all the same: its weight may then be in a file or not, and is not used."""
        self.mixer = build_part(MIXERS, mixer)
        self.ffn = build_part(FEED_FORWARDS, feed_forward) if feed_forward is not None else None
        self.mixer_norm = build_part(NORMS, mixer_norm)
        self.ffn_norm = build_part(NORMS, ffn_norm) if ffn_norm is not None else None
        if self.ffn is not None and self.ffn_norm is None:
            raise ValueError("a feed-forward needs the norm ahead of it")

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in self.parts())

    def parts(self):
        return tuple(p for p in (self.mixer_norm, self.mixer) + ((self.ffn_norm, self.ffn) if self.ffn is not None else ()))

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [s for p in self.parts() for s in p.tensor_specs()]
        if self.ffn is None and self.ffn_norm is not None:
            specs += [dataclasses.replace(s, optional=True) for s in self.ffn_norm.tensor_specs()]
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        for p in self.parts():
            p.bind(tensors, env)

    takes_next_norm = True

    @property
    def first_norm(self):
        return self.mixer_norm

    @staticmethod
    def _normed(norm, x: torch.Tensor, pending, ctx: StepContext, consumer):
        """The rows for `consumer`: normalised now, or left for it to normalise where it can."""
        if hasattr(pending, "settle"):  # a pending object of another block's own kind: it adds itself
            pending = pending.settle(x, ctx)
        if isinstance(pending, RowStats):
            if consumer.takes_normed_rows and pending.norm is norm and pending.scaled is not None:
                return NormedRows(x, norm, pending)
            return norm.forward(x, ctx)
        return norm.forward(x, ctx, delta=pending)

    def forward(self, x: torch.Tensor, pending, ctx: StepContext, cache: Optional[LayerCache], next_norm=None):
        h = self._normed(self.mixer_norm, x, pending, ctx, self.mixer)
        if self.mixer.takes_residual_sink:
            sink = ResidualSink(x, self.ffn_norm if self.ffn is not None else next_norm)
            pending = self.mixer.forward(h, ctx, cache, sink=sink)
            pending = sink.stats if pending is None else pending
        else:
            pending = self.mixer.forward(h, ctx, cache)
        if self.ffn is None:
            return pending
        h = self._normed(self.ffn_norm, x, pending, ctx, self.ffn)
        if self.ffn.takes_residual_sink:
            sink = ResidualSink(x, next_norm)
            pending = self.ffn.forward(h, ctx, sink=sink)
            return sink.stats if pending is None else pending
        return self.ffn.forward(h, ctx)


class ScaledDelta:
    """What a `ParallelBlock` leaves pending: the stream is x + scale * (sum of `pieces` [n, rows, width]).
    A consumer that cannot add it on its way calls `settle`, which brings x up to date."""

    def __init__(self, pieces: torch.Tensor, scale: float) -> None:
        self.pieces, self.scale = pieces, scale

    def settle(self, x: torch.Tensor, ctx: StepContext) -> None:
        ctx.kernels.add_scaled(x, self.pieces, self.scale)
        return None


@BLOCKS.register("parallel")
class ParallelBlock(Block):
    """One norm, whose output both sub-layers read: x += scale * (mixer(norm(x)) + ffn(norm(x))).  The
    feed-forward may be absent (`feed_forward=None`).  The add rides on the next block's norm where that
    norm takes a scaled delta (`takes_delta_scale`); otherwise the block adds before it returns."""

    takes_next_norm = True

    def __init__(self, mixer: PartSpec, norm: PartSpec, feed_forward: Optional[PartSpec] = None,
                 scale: float = 1.0) -> None:
        self.mixer = build_part(MIXERS, mixer)
        self.ffn = build_part(FEED_FORWARDS, feed_forward) if feed_forward is not None else None
        self.norm = build_part(NORMS, norm)
        self.scale = float(scale)

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in self.parts())

    @property
    def first_norm(self):
        return self.norm

    def parts(self):
        return tuple(p for p in (self.norm, self.mixer, self.ffn) if p is not None)

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        for p in self.parts():
            p.bind(tensors, env)

    def forward(self, x: torch.Tensor, pending, ctx: StepContext, cache: Optional[LayerCache], next_norm=None):
        kn = ctx.kernels
        if isinstance(pending, ScaledDelta) and getattr(self.norm, "takes_delta_scale", False):
            h = self.norm.forward(x, ctx, delta=pending.pieces, delta_scale=pending.scale)
        else:
            if hasattr(pending, "settle"):
                pending = pending.settle(x, ctx)
            h = self.norm.forward(x, ctx, delta=None if isinstance(pending, RowStats) else pending)
        subs = [(self.mixer, (h, ctx, cache))] + ([(self.ffn, (h, ctx))] if self.ffn is not None else [])
        pieces = ctx.ws.alloc((len(subs), x.shape[0], x.shape[1]), torch.float32)
        for i, (part, args) in enumerate(subs):
            if part.takes_out:
                part.forward(*args, out=pieces[i])
            else:  # a part that returns its result, whole or as pieces of its own
                self._copy_into(kn, part.forward(*args), pieces[i])
        # whoever looks at the stream between blocks (`ctx.observe`), and a norm that takes no scaled delta,
        # gets the stream whole
        if ctx.observe is None and next_norm is not None and getattr(next_norm, "takes_delta_scale", False):
            return ScaledDelta(pieces, self.scale)
        kn.add_scaled(x, pieces, self.scale)
        return None

    @staticmethod
    def _copy_into(kn, got: torch.Tensor, out: torch.Tensor) -> None:
        """A part's own result, whole [rows, width] or pieces [n, rows, width], summed into `out`."""
        if got.dim() == 3:
            kn.cast(got[0], out)
            for piece in got[1:]:
                kn.add(out, piece)
        else:
            kn.cast(got, out)


class RoundedStream:
    """What an `OutputNormBlock` leaves pending: the stream x is up to date, and `rounded` holds it in the run's
    dtype, made by the kernel that added the last sublayer's result.  The next block of the same kind reads it
    instead of rounding x again; anyone else has nothing to add (`settle`)."""

    def __init__(self, rounded: torch.Tensor) -> None:
        self.rounded = rounded

    def settle(self, x: torch.Tensor, ctx: StepContext) -> None:
        return None


@BLOCKS.register("output_norm")
class OutputNormBlock(Block):
    """Norms on the sublayers' results, none on their inputs: x += norm1(mixer(x)); x += norm2(ffn(x)).  The
    sublayers read the stream itself (rounded to the run's dtype where that is narrower).  The norms are RMS norms;
    one kernel normalises a sublayer's result, adds it to the 32-bit stream and leaves the stream's rounding for the
    next reader.  The feed-forward may be absent (`feed_forward=None`; then there is no second norm either)."""

    def __init__(self, mixer: PartSpec, mixer_norm: PartSpec, feed_forward: Optional[PartSpec] = None,
                 ffn_norm: Optional[PartSpec] = None) -> None:
        self.mixer = build_part(MIXERS, mixer)
        self.mixer_norm = build_part(NORMS, mixer_norm)
        self.ffn = build_part(FEED_FORWARDS, feed_forward) if feed_forward is not None else None
        self.ffn_norm = build_part(NORMS, ffn_norm) if feed_forward is not None else None
        if feed_forward is not None and ffn_norm is None:
            raise ValueError("a feed-forward needs the norm of its result")
        # the norm of a feed-forward that is not there: a file may hold its weight all the same; it is not used
        self.idle_norm = build_part(NORMS, ffn_norm) if feed_forward is None and ffn_norm is not None else None
        for norm in (self.mixer_norm, self.ffn_norm):
            if norm is not None and not getattr(norm, "deferrable", False):
                raise ValueError("the norms on the sublayers' results must be RMS norms")

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in self.parts())

    def parts(self):
        return tuple(p for p in (self.mixer, self.mixer_norm, self.ffn, self.ffn_norm) if p is not None)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [s for p in self.parts() for s in p.tensor_specs()]
        if self.idle_norm is not None:
            specs += [dataclasses.replace(s, optional=True) for s in self.idle_norm.tensor_specs()]
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        for p in self.parts():
            p.bind(tensors, env)

    @staticmethod
    def _run(part, args, ctx: StepContext, width: int) -> torch.Tensor:
        """A sublayer's result, whole [rows, width] in 32-bit."""
        rows = args[0].shape[0]
        if part.takes_out:
            out = ctx.ws.alloc((rows, width), torch.float32)
            part.forward(*args, out=out)
            return out
        got = part.forward(*args)
        if got.dim() == 3 or got.dtype != torch.float32:
            out = ctx.ws.alloc((rows, width), torch.float32)
            ParallelBlock._copy_into(ctx.kernels, got, out)
            return out
        return got

    def _add_normed(self, x, y, norm, ctx: StepContext):
        """x += norm(y); -> x in the run's dtype."""
        narrow = ctx.dtype != torch.float32
        rounded = ctx.ws.alloc(x.shape, ctx.dtype) if narrow else None
        ctx.kernels.rmsnorm_residual(x, y, norm.weight, norm.eps, rounded)
        return rounded if narrow else x

    def forward(self, x: torch.Tensor, pending, ctx: StepContext, cache: Optional[LayerCache]):
        kn = ctx.kernels
        if isinstance(pending, RoundedStream):
            h = pending.rounded
        else:
            if hasattr(pending, "settle"):
                pending = pending.settle(x, ctx)
            if pending is not None and not isinstance(pending, RowStats):
                kn.add(x, pending)
            h = x
            if ctx.dtype != torch.float32:
                h = ctx.ws.alloc(x.shape, ctx.dtype)
                kn.cast(x, h)
        h = self._add_normed(x, self._run(self.mixer, (h, ctx, cache), ctx, x.shape[1]), self.mixer_norm, ctx)
        if self.ffn is not None:
            h = self._add_normed(x, self._run(self.ffn, (h, ctx), ctx, x.shape[1]), self.ffn_norm, ctx)
        return RoundedStream(h) if h is not x else None


class NormedAhead:
    """What a `SandwichNormBlock` leaves pending: the stream x is up to date, and `normed` holds `norm` applied to it
    (the norm that the stream meets next), made by the kernel that added the block's last result.  A reader whose
    norm it is takes `normed`; anyone else has nothing to add (`settle`).  `added_extra`: the kernel also added what
    the model wants added ahead of the next run."""

    def __init__(self, normed: Optional[torch.Tensor], norm, added_extra: bool = False) -> None:
        self.normed, self.norm, self.added_extra = normed, norm, added_extra

    def settle(self, x: torch.Tensor, ctx: StepContext) -> None:
        return None


@BLOCKS.register("sandwich_norm")
class SandwichNormBlock(Block):
    """A norm ahead of every sublayer and one on its result: x += norm1b(mixer(norm1(x))); x += norm2b(ffn(norm2(x))).
    All four are RMS norms.  One kernel takes a sublayer's result (the sum of its pieces, each with its scale: two
    mixers side by side, routed experts beside a shared one), norms it, adds it to the 32-bit stream and applies the
    norm that the stream meets next: the feed-forward's, or the next block's first.  The feed-forward may be absent
    (`feed_forward=None`; its two norms' weights may then be in a file or not, and are not used)."""

    takes_next_norm = True
    takes_next_extra = True  # forward(..., next_extra=t): t is added to the stream after the block's last result

    def __init__(self, mixer: PartSpec, mixer_norm: PartSpec, mixer_out_norm: PartSpec,
                 feed_forward: Optional[PartSpec] = None, ffn_norm: Optional[PartSpec] = None,
                 ffn_out_norm: Optional[PartSpec] = None) -> None:
        self.mixer = build_part(MIXERS, mixer)
        self.mixer_norm = build_part(NORMS, mixer_norm)
        self.mixer_out_norm = build_part(NORMS, mixer_out_norm)
        self.ffn = build_part(FEED_FORWARDS, feed_forward) if feed_forward is not None else None
        if self.ffn is not None and (ffn_norm is None or ffn_out_norm is None):
            raise ValueError("a feed-forward needs the norm ahead of it and the norm of its result")
        self.ffn_norm = build_part(NORMS, ffn_norm) if self.ffn is not None else None
        self.ffn_out_norm = build_part(NORMS, ffn_out_norm) if self.ffn is not None else None
        # the norms of a feed-forward that is not there: a file may hold their weights all the same; they are not used
        self.idle_norms = [build_part(NORMS, n) for n in (ffn_norm, ffn_out_norm) if self.ffn is None and n is not None]
        for norm in (self.mixer_norm, self.mixer_out_norm, self.ffn_norm, self.ffn_out_norm):
            if norm is not None and not getattr(norm, "deferrable", False):
                raise ValueError("the norms around the sublayers must be RMS norms")

    @property
    def graph_safe(self) -> bool:
        return all(p.graph_safe for p in self.parts())

    @property
    def first_norm(self):
        return self.mixer_norm

    def parts(self):
        return tuple(p for p in (self.mixer_norm, self.mixer, self.mixer_out_norm, self.ffn_norm, self.ffn,
                                 self.ffn_out_norm) if p is not None)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [s for p in self.parts() for s in p.tensor_specs()]
        for idle in self.idle_norms:
            specs += [dataclasses.replace(s, optional=True) for s in idle.tensor_specs()]
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        for p in self.parts():
            p.bind(tensors, env)

    @staticmethod
    def _result(part, args, ctx: StepContext, width: int):
        """A sublayer's result as (pieces [n, rows, width] or [rows, width] in 32-bit, the pieces' scales)."""
        in_pieces = getattr(part, "forward_pieces", None)
        if in_pieces is not None:
            return in_pieces(*args)
        rows = args[0].shape[0]
        if part.takes_out:
            out = ctx.ws.alloc((rows, width), torch.float32)
            part.forward(*args, out=out)
            return out, (1.0,)
        got = part.forward(*args)
        if got.dtype == torch.float32 and got.is_contiguous() and (got.dim() == 2 or got.shape[0] <= 4):
            return got, (1.0,) * (1 if got.dim() == 2 else got.shape[0])
        out = ctx.ws.alloc((rows, width), torch.float32)
        ParallelBlock._copy_into(ctx.kernels, got, out)
        return out, (1.0,)

    def forward(self, x: torch.Tensor, pending, ctx: StepContext, cache: Optional[LayerCache], next_norm=None,
                next_extra=None):
        kn = ctx.kernels
        if isinstance(pending, NormedAhead) and pending.norm is self.mixer_norm and pending.normed is not None:
            h = pending.normed
        else:
            if hasattr(pending, "settle"):
                pending = pending.settle(x, ctx)
            h = self.mixer_norm.forward(x, ctx, delta=None if isinstance(pending, RowStats) else pending)
        y, scales = self._result(self.mixer, (h, ctx, cache), ctx, x.shape[1])
        out_norm = self.mixer_out_norm
        if self.ffn is not None:
            h = ctx.ws.alloc(x.shape, ctx.dtype)
            kn.postnorm_residual(x, y, scales, out_norm.weight, out_norm.eps, next_weight=self.ffn_norm.weight,
                                 next_eps=self.ffn_norm.eps, h=h)
            y, scales = self._result(self.ffn, (h, ctx), ctx, x.shape[1])
            out_norm = self.ffn_out_norm
        # whoever looks at the stream between blocks (`ctx.observe`) sees it as this block leaves it
        extra = next_extra if ctx.observe is None else None
        ahead = next_norm if getattr(next_norm, "deferrable", False) else None
        h = ctx.ws.alloc(x.shape, ctx.dtype) if ahead is not None else None
        kn.postnorm_residual(x, y, scales, out_norm.weight, out_norm.eps, extra=extra,
                             next_weight=ahead.weight if ahead is not None else None,
                             next_eps=ahead.eps if ahead is not None else 0.0, h=h)
        if ahead is None and extra is None:
            return None
        return NormedAhead(h, ahead, added_extra=extra is not None)
