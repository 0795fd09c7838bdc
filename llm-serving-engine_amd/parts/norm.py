"""Normalisation parts."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .base import NORMS, Part, TensorSpec


@dataclass(frozen=True)
class RMSNormSpec:
    """`weight_name` is the tensor's name below the part's prefix (a model whose files call it otherwise says so).
    `weight_scale` multiplies the weight (float32) when the part is built: a constant that a model puts on the normed
    rows (a scale of the logits behind the last norm) costs nothing that way."""

    size: int
    eps: float
    weight_name: str = "weight"
    kind: str = "rmsnorm"
    weight_scale: float = 1.0


@NORMS.register("rmsnorm")
class RMSNorm(Part):
    """y = x * rsqrt(mean(x^2) + eps) * weight (reference `model.py:14-23`), with
    the residual add in front of it: `hidden += delta` happens in the same
    kernel, in float32, and `hidden` stays float32 in every run dtype."""

    @classmethod
    def tensors(cls, spec: RMSNormSpec) -> dict[str, TensorSpec]:
        return {spec.weight_name: TensorSpec((spec.size,), role="norm")}

    def __init__(self, spec: RMSNormSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        self.weight = tensors[spec.weight_name]
        if spec.weight_scale != 1.0:
            self.weight = (self.weight.float() * float(spec.weight_scale)).contiguous()

    def forward(self, hidden: torch.Tensor, delta: torch.Tensor | None) -> torch.Tensor:
        """Adds `delta` into `hidden` (in place) and returns the normed rows in the run dtype."""
        return self.kernels.add_rms_norm(hidden, delta, self.weight, self.spec.eps)

    def add_normed(self, hidden: torch.Tensor, update: torch.Tensor) -> torch.Tensor:
        """The norm on a sublayer's output instead of its input: `hidden += update * rsqrt(mean(update^2) + eps) *
        weight` in place (float32; `update` may be partial sums, which are added first), and returns the new stream in
        the run dtype, as the next sublayer reads it."""
        return self.kernels.add_normed(hidden, update, self.weight, self.spec.eps)


@dataclass(frozen=True)
class LayerNormSpec:
    """`weight_name` and `bias_name` are the tensors' names below the part's prefix (a model whose files
    call them otherwise says so here)."""

    size: int
    eps: float
    weight_name: str = "weight"
    bias_name: str = "bias"
    kind: str = "layernorm"


@NORMS.register("layernorm")
class LayerNorm(Part):
    """y = (x - mean(x)) * rsqrt(mean((x - mean(x))^2) + eps) * weight + bias, all in float32, with the
    residual add in front of it as in `RMSNorm`."""

    @classmethod
    def tensors(cls, spec: LayerNormSpec) -> dict[str, TensorSpec]:
        return {spec.weight_name: TensorSpec((spec.size,), role="norm"), spec.bias_name: TensorSpec((spec.size,), role="bias")}

    def __init__(self, spec: LayerNormSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        self.weight = tensors[spec.weight_name]
        self.bias = tensors[spec.bias_name]

    def forward(self, hidden: torch.Tensor, delta: torch.Tensor | None) -> torch.Tensor:
        """Adds `delta` into `hidden` (in place) and returns the normed rows in the run dtype."""
        return self.kernels.add_layer_norm(hidden, delta, self.weight, self.bias, self.spec.eps)
