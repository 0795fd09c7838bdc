"""A recurrent mixer: linear attention over a matrix state per head that fades by a fixed factor a token."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .attention import Mixer
from .base import MIXERS, FixedState, TensorSpec
from .position import rotary_frequencies


@dataclass(frozen=True)
class DecayAttentionSpec:
    """`num_heads` heads with queries and keys of `dim` and values of `vdim`; `decays` one factor a head;
    `activation` on the three projections ("silu" or "none"); `eps` of the norm over the read-outs; `gate` squashes the gate
    ("sigmoid" or "silu").  `norm`: "row" (the heads' read-outs normed together, a weight as long as they) or "head" (every
    head's read-out by itself, one weight of vdim for all heads); `norm_weight` False: the norm has no weight and no tensor.
    `rot_dims`: the first so many dimensions of every query and key head turn by the position in pairs (`pairing`
    "adjacent": (2i, 2i + 1); "half": (i, i + rot_dims / 2)) with frequencies theta^(-2i / rot_dims), in float32; 0:
    positions do not enter.  `key_scale` multiplies the keys (after the rotation)."""

    hidden_size: int
    num_heads: int
    dim: int
    vdim: int
    decays: tuple[float, ...]
    eps: float
    activation: str = "silu"
    gate: str = "sigmoid"
    norm: str = "row"
    norm_weight: bool = True
    rot_dims: int = 0
    theta: float = 10000.0
    pairing: str = "half"
    key_scale: float = 1.0
    kind: str = "decay_attention"


@MIXERS.register("decay_attention")
class DecayAttention(Mixer):
    """q, k, v = act(W x) head by head; token by token, per head, with S [dim, vdim] from zero:

        S = decay S + k v^T;   o = S^T q

    then the heads' o side by side / their root mean square * norm * gate(W_g x), and W_o.  S, the decays, the
    scores q . k inside a run of tokens and the read-out are float32.  Per request the cache keeps S in a state slot
    that is zero when a request begins."""

    @classmethod
    def tensors(cls, spec: DecayAttentionSpec) -> dict[str, TensorSpec]:
        qk, v = spec.num_heads * spec.dim, spec.num_heads * spec.vdim
        found = {
            "q": TensorSpec((qk, spec.hidden_size)),
            "k": TensorSpec((qk, spec.hidden_size)),
            "v": TensorSpec((v, spec.hidden_size)),
            "g": TensorSpec((v, spec.hidden_size)),
            "o": TensorSpec((spec.hidden_size, v)),
        }
        if spec.norm_weight:
            found["norm"] = TensorSpec((v if spec.norm == "row" else spec.vdim,), role="norm")
        return found

    @classmethod
    def cache_need(cls, spec: DecayAttentionSpec) -> FixedState:
        return FixedState((spec.num_heads, spec.dim, spec.vdim))

    def __init__(self, spec: DecayAttentionSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        if len(spec.decays) != spec.num_heads:
            raise ValueError("decay attention: one decay a head")
        if spec.norm not in ("row", "head") or spec.pairing not in ("adjacent", "half"):
            raise ValueError("decay attention: norm is 'row' or 'head', pairing 'adjacent' or 'half'")
        if spec.rot_dims % 2 or spec.rot_dims > spec.dim:
            raise ValueError("decay attention: the rotated dimensions are an even number within dim")
        self.inputs = kernels.prepare_linear([tensors[name] for name in ("q", "k", "v", "g")], None)
        self.decays = kernels.to_device(torch.tensor(spec.decays, dtype=torch.float64).to(torch.float32))
        normed = spec.num_heads * spec.vdim if spec.norm == "row" else spec.vdim
        self.norm = tensors["norm"] if spec.norm_weight else kernels.to_device(torch.ones((normed,), dtype=torch.float32))
        self.out = kernels.prepare_linear([tensors["o"]], None)
        self.turned = spec.rot_dims > 0 or spec.key_scale != 1.0
        self.frequencies = None
        if spec.rot_dims:
            shared = kernels.__dict__.setdefault("_rotary_frequencies", {})
            key = (spec.rot_dims, spec.theta, None)
            if key not in shared:
                frequencies, magnitude = rotary_frequencies(spec.rot_dims, spec.theta, None)
                shared[key] = (kernels.to_device(frequencies), magnitude)
            self.frequencies = shared[key][0]

    def forward(self, x: torch.Tensor, batch, cell) -> torch.Tensor:
        kernels, spec = self.kernels, self.spec
        heads, qk, v = spec.num_heads, spec.num_heads * spec.dim, spec.num_heads * spec.vdim
        # Where the queries and keys are turned they stay float32 from the product to the state: what enters the
        # recurrence is rounded nowhere between.
        projected = kernels.linear(x, self.inputs, out_dtype=torch.float32 if self.turned else None)  # [T, q | k | v | g]
        if self.turned:
            table = kernels.rotary_table(batch, self.frequencies) if spec.rot_dims else None
            # (queries and keys lie side by side: one call, the keys scaled)
            kernels.rotate_heads(projected, 0, spec.dim, 2 * heads, table, spec.rot_dims, spec.pairing, spec.key_scale, scale_from=heads)
        read = kernels.decay_attention(
            projected, 0, qk, 2 * qk, heads, spec.dim, spec.vdim, self.decays, spec.activation, batch, cell.state
        )  # float32 [T, heads * vdim]
        if spec.norm == "row":  # one norm over all heads: a single "head" as wide as the row
            gated = kernels.gated_head_norm(read, projected, 2 * qk + v, self.norm, spec.eps, 1, v, spec.gate)
        else:
            gated = kernels.gated_head_norm(read, projected, 2 * qk + v, self.norm, spec.eps, heads, spec.vdim, spec.gate)
        return kernels.linear(gated, self.out, out_dtype=torch.float32, partial=True)
