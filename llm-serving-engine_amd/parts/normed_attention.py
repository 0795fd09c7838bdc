"""Attention over a sliding window whose queries and keys are normed, with the options some designs put around
it: heads rotated in part, capped scores, a sink in the softmax's denominator, values blended with an earlier
layer's, and a gate a head on the result."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .attention import Mixer
from .base import MIXERS, PagedKeyValue, TensorSpec
from .position import HeadLayout, LinearScaling, WavelengthScaling, YarnScaling, rotary_frequencies


@dataclass(frozen=True)
class NormedAttentionSpec:
    """`num_heads` query heads and `num_kv_heads` key/value heads (query head h reads key/value head h // (heads /
    kv_heads)); queries and keys of `dim`, values of `vdim`.

    `norm`: "head" (RMS norm of every query and key head with one weight of `dim` for all heads), "row" (RMS norm of
    the whole query projection and of the whole key projection, with weights as long as they), or None.
    `rot_dims`: the first so many dimensions of every query and key head turn by the position, in adjacent pairs
    (2i, 2i + 1) or, with `pairing` "half", in pairs (i, i + rot_dims / 2), with the frequencies theta^(-2i / rot_dims)
    stretched by `scaling`; 0: positions do not enter.
    `soft_cap`: scores become cap * tanh(score / cap).  `sink`: a learned number a head whose exponential is added
    once to the softmax's denominator.  `gate`: head h's result times sigmoid of row h of a product of the mixer's input.
    `values`: None, "give" (the step's values are shown to later layers under `values_name`) or "take" (v <- (1 - a) v
    + a v_given with the learned number a; the blended v is what is cached).
    `keep_first`: under a window, the first so many tokens of a sequence stay visible to every later query, at their
    own positions (a query at p sees the keys at j <= p with p - j < window or j < keep_first)."""

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    dim: int
    vdim: int
    scale: float
    eps: float
    window: int | None = None
    bias: bool = False
    norm: str | None = "head"
    rot_dims: int = 0
    theta: float = 10000.0
    scaling: YarnScaling | WavelengthScaling | LinearScaling | None = None
    pairing: str = "adjacent"
    soft_cap: float | None = None
    sink: bool = False
    gate: bool = False
    values: str | None = None
    values_name: str = "values"
    keep_first: int = 0
    kind: str = "normed_attention"

    @property
    def head_width(self) -> int:
        """What a head takes in the cache and in the attention kernels: keys and values side by side have one width
        there, the larger of the two rounded up to a multiple of 16, the rest of a narrower head zeros."""
        return -(-max(self.dim, self.vdim) // 16) * 16


@MIXERS.register("normed_attention")
class NormedAttention(Mixer):
    """q = W_q x (+ b), k, v likewise; norm; rotation; v blended; per head softmax over the keys of the last
    `window` positions of (q . k) * scale, capped, with the sink; the gate; W_o.

    The heads go to the engine's paged attention as rows of `head_width`: a key's or value's columns beyond its own
    size are zeros, which change neither a score nor a result's own columns, and the output projection's weight has
    zero columns where the results do.  Norms, angles, cosines and sines, the blend and the gate are float32."""

    @classmethod
    def tensors(cls, spec: NormedAttentionSpec) -> dict[str, TensorSpec]:
        q_size, k_size, v_size = spec.num_heads * spec.dim, spec.num_kv_heads * spec.dim, spec.num_kv_heads * spec.vdim
        found = {
            "q": TensorSpec((q_size, spec.hidden_size)),
            "k": TensorSpec((k_size, spec.hidden_size)),
            "v": TensorSpec((v_size, spec.hidden_size)),
            "o": TensorSpec((spec.hidden_size, spec.num_heads * spec.vdim)),
        }
        if spec.bias:
            found.update({"q.b": TensorSpec((q_size,), role="bias"), "k.b": TensorSpec((k_size,), role="bias"), "v.b": TensorSpec((v_size,), role="bias")})
        if spec.norm == "head":
            found.update({"q.norm": TensorSpec((spec.dim,), role="norm"), "k.norm": TensorSpec((spec.dim,), role="norm")})
        elif spec.norm == "row":
            found.update({"q.norm": TensorSpec((q_size,), role="norm"), "k.norm": TensorSpec((k_size,), role="norm")})
        if spec.values is not None:
            found["vmix"] = TensorSpec((), role="bias")  # (a layer that gives its values has the number too, and does not use it)
        if spec.sink:
            found["sink"] = TensorSpec((spec.num_heads,), role="bias")
        if spec.gate:
            found["g"] = TensorSpec((spec.num_heads, spec.hidden_size))
        return found

    @classmethod
    def cache_need(cls, spec: NormedAttentionSpec) -> PagedKeyValue:
        return PagedKeyValue(spec.num_kv_heads, spec.head_width, spec.window, spec.keep_first if spec.window is not None else 0)

    def __init__(self, spec: NormedAttentionSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        if spec.num_heads % spec.num_kv_heads:
            raise ValueError("normed attention: the query heads are a multiple of the key/value heads")
        if spec.norm not in (None, "head", "row") or spec.values not in (None, "give", "take"):
            raise ValueError("normed attention: norm is 'head', 'row' or None; values 'give', 'take' or None")
        if spec.pairing not in ("adjacent", "half"):
            raise ValueError("normed attention: pairing is 'adjacent' or 'half'")
        if spec.rot_dims % 2 or spec.rot_dims > spec.dim:
            raise ValueError("normed attention: the rotated dimensions are an even number within dim")
        if spec.keep_first < 0:
            raise ValueError("normed attention: keep_first counts tokens")
        self.keep_first = spec.keep_first if spec.window is not None else 0
        heads, width = spec.num_heads, spec.head_width
        self.layout = HeadLayout(heads, spec.num_kv_heads, width)
        names = ["q", "k", "v"] + (["g"] if spec.gate else [])
        biases = None
        if spec.bias:
            biases = [tensors["q.b"], tensors["k.b"], tensors["v.b"]]
            if spec.gate:
                biases.append(torch.zeros((heads,), dtype=biases[0].dtype, device=biases[0].device))
        self.inputs = kernels.prepare_linear([tensors[name] for name in names], biases)  # [q | k | v | gates]
        self.q_norm = tensors.get("q.norm") if spec.norm else None
        self.k_norm = tensors.get("k.norm") if spec.norm else None
        self.blend = float(tensors["vmix"].float()) if spec.values == "take" else 0.0
        self.sinks = kernels.to_device(tensors["sink"].float().contiguous()) if spec.sink else None
        out = tensors["o"]
        if width != spec.vdim:  # the results' columns beyond vdim are zeros: the weight gets columns for them
            wide = torch.zeros((spec.hidden_size, heads, width), dtype=out.dtype, device=out.device)
            wide[:, :, : spec.vdim] = out.view(spec.hidden_size, heads, spec.vdim)
            out = wide.view(spec.hidden_size, heads * width)
        self.out = kernels.prepare_linear([out.contiguous()], None)
        self.frequencies = None
        if spec.rot_dims:
            shared = kernels.__dict__.setdefault("_rotary_frequencies", {})
            key = (spec.rot_dims, spec.theta, spec.scaling)
            if key not in shared:
                frequencies, magnitude = rotary_frequencies(spec.rot_dims, spec.theta, spec.scaling)
                shared[key] = (kernels.to_device(frequencies), magnitude)
            self.frequencies, self.magnitude = shared[key]

    def forward(self, x: torch.Tensor, batch, cell) -> torch.Tensor:
        kernels, spec = self.kernels, self.spec
        q_size, k_size, v_size = spec.num_heads * spec.dim, spec.num_kv_heads * spec.dim, spec.num_kv_heads * spec.vdim
        projected = kernels.linear(x, self.inputs)  # [T, q | k | v | gates]
        given = None
        if spec.values == "give":
            batch.computed[("given values", spec.values_name)] = (projected, q_size + k_size, v_size)
        elif spec.values == "take":
            given = batch.computed.get(("given values", spec.values_name))
            if given is None or given[2] != v_size:
                raise RuntimeError("normed attention: no earlier layer of this step gave values of this size")
        table = kernels.rotary_table(batch, self.frequencies, self.magnitude) if spec.rot_dims else None
        # per token the heads' queries, keys and values as the attention reads them: normed, turned, blended, widened
        plain = spec.soft_cap is None and self.sinks is None and not spec.gate and not self.keep_first
        rows = kernels.assemble_heads(
            projected, 0, q_size, q_size + k_size, spec.num_heads, spec.num_kv_heads, spec.dim, spec.vdim, spec.head_width,
            spec.norm, self.q_norm, self.k_norm, spec.eps, table, spec.rot_dims,
            given[0] if given else None, given[1] if given else 0, self.blend,
            batch=batch, cell=None if plain else cell,  # (with plain scores the attention below stores, and may fuse that)
            pairing=spec.pairing,
        )
        if plain:
            return kernels.rotate_store_attend(rows, self.layout, batch, cell, None, "none", spec.scale, spec.window, project=self.out)
        mixed = kernels.paged_attention(
            rows, self.layout, batch, cell, spec.scale, spec.window, soft_cap=spec.soft_cap, sinks=self.sinks, keep_first=self.keep_first,
        )
        if spec.gate:
            kernels.scale_heads(mixed, spec.num_heads, spec.head_width, projected, q_size + k_size + v_size, "sigmoid")
        return kernels.linear(mixed, self.out, out_dtype=torch.float32, partial=True)
