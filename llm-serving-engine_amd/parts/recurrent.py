"""A recurrent mixer with a diagonal state: a gated linear recurrence behind a short causal convolution, beside a
gelu branch that gates what is read out (the recurrent block of Griffin-style models)."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .attention import Mixer
from .base import MIXERS, FixedState, TensorSpec


@dataclass(frozen=True)
class GatedRecurrenceSpec:
    """Two branches of `width`; the gates' products are block-diagonal in `blocks` equal parts; `taps` of the
    convolution; `rate` is the constant c of log a = -c r softplus(lam)."""

    hidden_size: int
    width: int
    blocks: int
    taps: int
    rate: float = 8.0
    kind: str = "gated_recurrence"


@MIXERS.register("gated_recurrence")
class GatedRecurrence(Mixer):
    """y = gelu_tanh(W_y x + b_y); u = conv(W_x x + b_x) + b_conv per channel over the last `taps` tokens; in each
    of the `blocks` parts of u: r = sigmoid(R_b u_b + b_r), i = sigmoid(I_b u_b + b_i); a = exp(-rate r softplus(lam));
    S <- a S + sqrt(1 - a^2) i u, from S = 0; the result is W_o (S y).  Gates, decays and S are float32.  Per
    request the cache keeps S and the convolution's last `taps - 1` inputs, zero when a request begins."""

    @classmethod
    def tensors(cls, spec: GatedRecurrenceSpec) -> dict[str, TensorSpec]:
        part = spec.width // spec.blocks
        return {
            "y": TensorSpec((spec.width, spec.hidden_size)),
            "y.b": TensorSpec((spec.width,), role="bias"),
            "x": TensorSpec((spec.width, spec.hidden_size)),
            "x.b": TensorSpec((spec.width,), role="bias"),
            "conv": TensorSpec((spec.width, spec.taps)),
            "conv.b": TensorSpec((spec.width,), role="bias"),
            "ra": TensorSpec((spec.blocks, part, part)),
            "ra.b": TensorSpec((spec.blocks, part), role="bias"),
            "ri": TensorSpec((spec.blocks, part, part)),
            "ri.b": TensorSpec((spec.blocks, part), role="bias"),
            "lam": TensorSpec((spec.width,), role="bias"),
            "o": TensorSpec((spec.hidden_size, spec.width)),
        }

    @classmethod
    def cache_need(cls, spec: GatedRecurrenceSpec) -> dict[str, FixedState]:
        need = {"state": FixedState((spec.width,))}
        if spec.taps > 1:
            need["window"] = FixedState((spec.taps - 1, spec.width))
        return need

    def __init__(self, spec: GatedRecurrenceSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        if spec.width % spec.blocks:
            raise ValueError("gated recurrence: the width is a multiple of the blocks")
        self.inputs = kernels.prepare_linear([tensors["x"], tensors["y"]], [tensors["x.b"], tensors["y.b"]])  # [x | y]
        self.taps = kernels.to_device(tensors["conv"].float().contiguous())
        self.conv_bias = kernels.to_device(tensors["conv.b"].float().contiguous())
        # a block's two gate matrices one above the other: one product per block gives [r_b | i_b]
        self.gates = kernels.prepare_headwise_linear(torch.cat([tensors["ra"], tensors["ri"]], dim=1).contiguous())
        self.gate_bias = kernels.to_device(torch.cat([tensors["ra.b"], tensors["ri.b"]], dim=1).float().contiguous())  # [blocks, 2 part]
        lam = tensors["lam"].float()
        self.rates = kernels.to_device((-spec.rate * torch.nn.functional.softplus(lam)).contiguous())  # log a = rates * r
        self.out = kernels.prepare_linear([tensors["o"]], None)

    def forward(self, x: torch.Tensor, batch, cell) -> torch.Tensor:
        kernels, spec = self.kernels, self.spec
        projected = kernels.linear(x, self.inputs)  # [T, x | y]
        window = cell["window"].state if "window" in cell else None
        u = kernels.causal_conv(projected, spec.width, self.taps, "none", batch, window, bias=self.conv_bias)  # [T, width]
        gates = kernels.headwise_linear(u, 0, spec.width // spec.blocks, self.gates)  # [T, blocks * (r_b | i_b)]
        read = kernels.gated_recurrence(
            u, gates, self.gate_bias, self.rates, projected, spec.width, "gelu_tanh", spec.blocks, batch, cell["state"].state
        )  # run dtype [T, width]: S * act(y)
        return kernels.linear(read, self.out, out_dtype=torch.float32, partial=True)
