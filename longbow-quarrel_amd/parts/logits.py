"""Steps on the logits after the head."""
from __future__ import annotations

import torch

from .base import LOGIT_STEPS, LogitsStep, StepContext


@LOGIT_STEPS.register("scale")
class ScaleLogits(LogitsStep):
    """logits *= factor, a model's own constant (taken in 32-bit, on the 32-bit logits)."""

    graph_safe = True

    def __init__(self, factor: float) -> None:
        self.factor = float(factor)

    def forward(self, logits: torch.Tensor, ctx: StepContext) -> None:
        if self.factor != 1.0:
            ctx.kernels.scale(logits, self.factor)
