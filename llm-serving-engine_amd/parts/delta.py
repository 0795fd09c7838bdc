"""A recurrent mixer: the gated delta rule over a matrix state per head, behind short causal convolutions."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .attention import Mixer
from .base import MIXERS, FixedState, TensorSpec


@dataclass(frozen=True)
class GatedDeltaSpec:
    """`num_heads` value heads of `vdim`, `num_kv_heads` query/key heads of `dim` (value head h reads
    query/key head h // (num_heads / num_kv_heads)); `taps` of the convolutions; `eps` of the output norm.

    `decay`: "head" (one decay a head and token, from `a` [heads, hidden] and `dt_bias` [heads]) or "channel" (one a head
    and key channel, from a product of two low-rank factors `a1` [decay_rank, hidden], `a2` [heads * dim, decay_rank] and
    `dt_bias` [heads * dim]).  `gate_rank`: None (the output gate is one product `g`) or the inner size of its two factors
    `g1`, `g2`.  `gate_activation`: what squashes the output gate (silu or sigmoid)."""

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    dim: int
    vdim: int
    taps: int
    eps: float
    decay: str = "head"
    decay_rank: int | None = None
    gate_rank: int | None = None
    gate_activation: str = "silu"
    kind: str = "gated_delta"

    @property
    def channels(self) -> int:
        """q, k and v side by side: what the convolutions run over."""
        return 2 * self.num_kv_heads * self.dim + self.num_heads * self.vdim


@MIXERS.register("gated_delta")
class GatedDelta(Mixer):
    """q, k, v = silu(conv(W x)) per channel over the last `taps` tokens; q and k made unit vectors per head
    (x / sqrt(sum x^2 + 1e-6)), q times dim^-1/2; per value head beta = sigmoid(W_b x) and the decay
    g = exp(-exp(A_log) softplus(W_a x + dt_bias)).  Token by token, per head, with S [dim, vdim]:

        S = g S;   u = beta (v - S^T k);   S = S + k u^T;   o = S^T q

    then o / rms(o) * norm * silu(W_g x) head by head, and W_o.  With a decay per key channel g is a vector of
    `dim` a head and scales the rows of S.  Decay, beta, the unit norms and S are float32.  Per request the cache keeps S (as S^T, [vdim, dim] a head) and the last `taps - 1` inputs of the
    convolutions, both in state slots that are zero when a request begins."""

    @classmethod
    def tensors(cls, spec: GatedDeltaSpec) -> dict[str, TensorSpec]:
        qk, v = spec.num_kv_heads * spec.dim, spec.num_heads * spec.vdim
        found = {
            "q": TensorSpec((qk, spec.hidden_size)),
            "q.conv": TensorSpec((qk, spec.taps)),
            "k": TensorSpec((qk, spec.hidden_size)),
            "k.conv": TensorSpec((qk, spec.taps)),
            "v": TensorSpec((v, spec.hidden_size)),
            "v.conv": TensorSpec((v, spec.taps)),
            "b": TensorSpec((spec.num_heads, spec.hidden_size)),
            "A_log": TensorSpec((spec.num_heads,), role="bias"),
            "norm": TensorSpec((spec.vdim,), role="norm"),
            "o": TensorSpec((spec.hidden_size, v)),
        }
        if spec.decay == "channel":
            found["a1"] = TensorSpec((cls._rank(spec.decay_rank, "decay_rank"), spec.hidden_size))
            found["a2"] = TensorSpec((spec.num_heads * spec.dim, spec.decay_rank))
            found["dt_bias"] = TensorSpec((spec.num_heads * spec.dim,), role="bias")
        else:
            found["a"] = TensorSpec((spec.num_heads, spec.hidden_size))
            found["dt_bias"] = TensorSpec((spec.num_heads,), role="bias")
        if spec.gate_rank is not None:
            found["g1"] = TensorSpec((spec.gate_rank, spec.hidden_size))
            found["g2"] = TensorSpec((v, spec.gate_rank))
        else:
            found["g"] = TensorSpec((v, spec.hidden_size))
        return found

    @staticmethod
    def _rank(rank, name: str) -> int:
        if rank is None:
            raise ValueError(f"gated delta: {name} is not given (a model folder's tensors give it)")
        return rank

    @classmethod
    def cache_need(cls, spec: GatedDeltaSpec) -> dict[str, FixedState]:
        need = {"state": FixedState((spec.num_heads, spec.vdim, spec.dim))}  # S transposed: a value dimension's column lies side by side
        if spec.taps > 1:
            need["window"] = FixedState((spec.taps - 1, spec.channels))
        return need

    def __init__(self, spec: GatedDeltaSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        if spec.num_heads % spec.num_kv_heads:
            raise ValueError("gated delta: the value heads are a multiple of the query/key heads")
        if spec.decay not in ("head", "channel") or spec.gate_activation not in ("silu", "sigmoid"):
            raise ValueError("gated delta: decay is 'head' or 'channel', the gate's activation silu or sigmoid")
        self.taps = kernels.to_device(torch.cat([tensors[name + ".conv"] for name in ("q", "k", "v")], dim=0).float().contiguous())
        self.rate = kernels.to_device(tensors["A_log"].float().contiguous())
        self.step_bias = kernels.to_device(tensors["dt_bias"].float().contiguous())
        self.norm = tensors["norm"]
        self.out = kernels.prepare_linear([tensors["o"]], None)
        self.factored = spec.decay == "channel" or spec.gate_rank is not None
        if not self.factored:
            # one product for what the convolutions and the output gate read, one (kept float32) for what enters the recurrence
            self.inputs = kernels.prepare_linear([tensors[name] for name in ("q", "k", "v", "g")], None)
            self.controls = kernels.prepare_linear([tensors["b"], tensors["a"]], None)
            return
        # With low-rank factors: what the convolutions read and the factors' first halves are one product; the second
        # halves are one more, over a weight with a block for each factor (zeros elsewhere), kept float32.
        first = [tensors[name] for name in ("q", "k", "v")]
        self.decay_rank = spec.decay_rank if spec.decay == "channel" else 0
        self.gate_rank = spec.gate_rank or 0
        low = ([tensors["a1"]] if self.decay_rank else []) + ([tensors["g1"]] if self.gate_rank else [])
        self.inputs = kernels.prepare_linear(first + ([] if self.gate_rank else [tensors["g"]]), None)
        self.low = kernels.prepare_linear(low, None)
        decay_rows = spec.num_heads * spec.dim if self.decay_rank else 0
        gate_rows = spec.num_heads * spec.vdim if self.gate_rank else 0
        second = torch.zeros((decay_rows + gate_rows, self.decay_rank + self.gate_rank), dtype=tensors["o"].dtype, device=tensors["o"].device)
        if self.decay_rank:
            second[:decay_rows, : self.decay_rank] = tensors["a2"]
        if self.gate_rank:
            second[decay_rows:, self.decay_rank :] = tensors["g2"]
        self.second = kernels.prepare_linear([second.contiguous()], None)
        self.controls = kernels.prepare_linear([tensors["b"]] + ([] if self.decay_rank else [tensors["a"]]), None)

    def forward(self, x: torch.Tensor, batch, cell) -> torch.Tensor:
        kernels, spec = self.kernels, self.spec
        projected = kernels.linear(x, self.inputs)  # [T, q | k | v (| g)]
        controls = kernels.linear(x, self.controls, out_dtype=torch.float32)  # [T, b (| a)]
        window = cell["window"].state if "window" in cell else None
        gates, gate_first = projected, spec.channels
        steps = None
        if self.factored:
            expanded = kernels.linear(kernels.linear(x, self.low), self.second, out_dtype=torch.float32)  # [T, a of heads * dim | g of heads * vdim]
            if self.decay_rank:
                steps = expanded
            if self.gate_rank:
                gates, gate_first = expanded, spec.num_heads * spec.dim if self.decay_rank else 0
        # the convolutions over [q | k | v], their silu, the unit vectors, the gates and the recurrence
        read = kernels.conv_gated_delta_rule(
            projected, spec.channels, self.taps, "silu", controls, self.rate, self.step_bias, spec.num_heads, spec.num_kv_heads,
            spec.dim, spec.vdim, batch, window, cell["state"].state, channel_steps=steps,
        )  # float32 [T, heads * vdim]
        gated = kernels.gated_head_norm(read, gates, gate_first, self.norm, spec.eps, spec.num_heads, spec.vdim, spec.gate_activation)
        return kernels.linear(gated, self.out, out_dtype=torch.float32, partial=True)
