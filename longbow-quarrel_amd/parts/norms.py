"""RMSNorm: y = x / sqrt(mean(x^2) + eps) * w, eps inside the root, the weight
after the normalisation (internal/device/kernels.metal:905-942; host twin
internal/device/cpu_ref.go:63-83).  Statistics in 32-bit, weight held in 32-bit
(internal/engine/engine.go:788-792 promotes norm weights the same way).
`offset`: the stored weight lies around zero and the norm multiplies by offset + w (a design that stores its gains
as 1 + w names offset = 1); the sum is made once, in 32-bit, when the weights are bound."""
from __future__ import annotations

from typing import List, Mapping, Optional

import torch

from .base import NORMS, VECTOR32, BuildEnv, Norm, StepContext, TensorSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True
    deferrable = True  # a consumer may apply it itself from x, weight, eps and the rows' sums of squares

    def __init__(self, width: int, eps: float, name: str, offset: float = 0.0) -> None:
        self.width = int(width)
        self.eps = float(eps)
        self.name = name
        self.offset = float(offset)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name, (self.width,), kind=VECTOR32, init="normal" if self.offset else "around_one")]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        w = tensors[self.name]
        self.weight = (w + self.offset if self.offset else w).contiguous()

    def forward(self, x: torch.Tensor, ctx: StepContext, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
        out = ctx.ws.alloc(x.shape, ctx.dtype)
        ctx.kernels.rmsnorm(x, self.weight, self.eps, out, delta=delta)
        return out


@NORMS.register("dynamic_tanh")
class DynamicTanh(Norm):
    """y = tanh(alpha x) w + b with a learned scalar alpha: an element-wise squashing in a norm's place, which
    computes no mean and no variance (Zhu, Chen, He, LeCun, Liu: "Transformers without Normalization").
    The tanh is taken in 32-bit.  `names` gives the tensors of the weight, the bias and alpha."""

    graph_safe = True
    deferrable = False  # there are no row statistics that a product could fold in
    takes_delta_scale = True  # forward(..., delta_scale=s) adds s * delta

    def __init__(self, width: int, name: str, bias_name: Optional[str] = None, alpha_name: Optional[str] = None) -> None:
        self.width = int(width)
        self.name = name
        self.bias_name = bias_name or name + ".b"
        self.alpha_name = alpha_name or name + ".alpha"
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None
        self.alpha: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name, (self.width,), kind=VECTOR32, init="around_one"),
                TensorSpec(self.bias_name, (self.width,), kind=VECTOR32, init="normal"),
                TensorSpec(self.alpha_name, (), kind=VECTOR32, init="around_one")]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        self.weight = tensors[self.name].contiguous()
        self.bias = tensors[self.bias_name].contiguous()
        self.alpha = tensors[self.alpha_name].reshape(1).contiguous()  # read on the device: no copy to the host

    def forward(self, x: torch.Tensor, ctx: StepContext, delta: Optional[torch.Tensor] = None,
                delta_scale: float = 1.0) -> torch.Tensor:
        out = ctx.ws.alloc(x.shape, ctx.dtype)
        ctx.kernels.dynamic_tanh(x, self.weight, self.bias, self.alpha, out, delta=delta, delta_scale=delta_scale)
        return out
