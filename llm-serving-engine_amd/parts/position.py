"""Position encodings that act on queries and keys before they are cached."""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch

from .base import POSITIONS, Part


@dataclass(frozen=True)
class HeadLayout:
    """How one token's projected row is laid out: q heads, then k heads, then v heads."""

    num_heads: int
    num_kv_heads: int
    head_dim: int

    @property
    def width(self) -> int:
        return (self.num_heads + 2 * self.num_kv_heads) * self.head_dim


@dataclass(frozen=True)
class RotarySpec:
    head_dim: int
    theta: float
    pairing: str = "half"  # "half": (j, j + D/2); "adjacent": (2j, 2j+1)
    kind: str = "rotary"


@dataclass(frozen=True)
class NoPositionSpec:
    kind: str = "none"


class PositionEncoding(Part):
    def encode_and_store(self, qkv, layout: HeadLayout, batch, cell) -> None:
        """Encodes q and k of `qkv` [T, layout.width] in place by each token's
        position and, if `cell` is writable, stores k and v in the cell's pages."""
        raise NotImplementedError

    def encode_store_attend(self, qkv, layout: HeadLayout, batch, cell, scale: float, window, project=None) -> "torch.Tensor":
        """`encode_and_store`, then attention over the cell's pages; with `project` (a prepared linear),
        then that product of the result, in float32, possibly as partial sums.  An encoding that a kernel
        can apply on the way (rotary) overrides this to let the kernel library fuse what it can."""
        self.encode_and_store(qkv, layout, batch, cell)
        mixed = self.kernels.paged_attention(qkv, layout, batch, cell, scale, window)
        if project is None:
            return mixed
        return self.kernels.linear(mixed, project, out_dtype=torch.float32, partial=True)


@POSITIONS.register("rotary")
class Rotary(PositionEncoding):
    """Reference `model.py:26-43`: inv[j] = theta^(-2j/D), angle = position *
    inv[j] in float32; the pair (a, b) becomes (a cos - b sin, b cos + a sin).
    The reference gathers cos/sin from a table built at start-up; here the
    kernel computes them from the position, in float32, so no length is fixed."""

    def __init__(self, spec: RotarySpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        if spec.pairing not in ("half", "adjacent"):
            raise ValueError(f"unknown rotary pairing {spec.pairing!r}")
        # one tensor per (head size, theta) and kernel library: layers that rotate alike share it,
        # and with it whatever the library derives from it per step
        shared = kernels.__dict__.setdefault("_rotary_frequencies", {})
        key = (spec.head_dim, spec.theta)
        if key not in shared:
            exponents = torch.arange(0, spec.head_dim, 2, dtype=torch.float32) / spec.head_dim
            shared[key] = kernels.to_device(1.0 / (spec.theta ** exponents))
        self.inverse_frequencies = shared[key]

    def encode_and_store(self, qkv, layout: HeadLayout, batch, cell) -> None:
        self.kernels.rotate_and_store(
            qkv, layout, batch, cell, self.inverse_frequencies, self.spec.pairing
        )

    def encode_store_attend(self, qkv, layout: HeadLayout, batch, cell, scale: float, window, project=None):
        return self.kernels.rotate_store_attend(
            qkv, layout, batch, cell, self.inverse_frequencies, self.spec.pairing, scale, window, project=project
        )


@POSITIONS.register("none")
class NoPosition(PositionEncoding):
    """No encoding: keys and values are only stored."""

    def encode_and_store(self, qkv, layout: HeadLayout, batch, cell) -> None:
        self.kernels.rotate_and_store(qkv, layout, batch, cell, None, "none")

    def encode_store_attend(self, qkv, layout: HeadLayout, batch, cell, scale: float, window, project=None):
        return self.kernels.rotate_store_attend(qkv, layout, batch, cell, None, "none", scale, window, project=project)


@dataclass(frozen=True)
class YarnScaling:
    """Frequencies stretched for contexts longer than the `original` one: a pair whose wavelength makes more
    than `fast` turns over the original context keeps its frequency, one that makes fewer than `slow` has it
    divided by `factor`, a linear ramp over the pair index between; cosines and sines grow by 0.1 ln(factor) + 1."""

    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class WavelengthScaling:
    """Frequencies stretched by wavelength: a pair whose wavelength is below `original / high` keeps its frequency,
    one above `original / low` has it divided by `factor`, and between the two the divided and the plain frequency
    are blended, s = (original / wavelength - low) / (high - low) of the plain one.  Cosines and sines stay as they are."""

    factor: float
    low: float
    high: float
    original: float


@dataclass(frozen=True)
class LinearScaling:
    """Every frequency divided by `factor` (positions counted in steps of 1 / factor).  Cosines and sines stay as they are."""

    factor: float


def rotary_frequencies(dims: int, theta: float, scaling: "YarnScaling | WavelengthScaling | LinearScaling | None" = None) -> tuple[torch.Tensor, float]:
    """(float32 frequencies [dims / 2] of pair i, theta^(-2i / dims), stretched by `scaling`; what the cosines
    and sines are multiplied by).  Computed in float64 and rounded once."""
    index = torch.arange(dims // 2, dtype=torch.float64)
    plain = float(theta) ** (-2.0 * index / dims)
    if scaling is None:
        return plain.to(torch.float32), 1.0
    if isinstance(scaling, LinearScaling):
        return (plain / float(scaling.factor)).to(torch.float32), 1.0
    if isinstance(scaling, WavelengthScaling):
        wavelength = 2.0 * math.pi / plain
        share = ((scaling.original / wavelength - scaling.low) / (scaling.high - scaling.low)).clamp(0.0, 1.0)
        blended = (1.0 - share) * plain / scaling.factor + share * plain
        stretched = torch.where(wavelength < scaling.original / scaling.high, plain,
                                torch.where(wavelength > scaling.original / scaling.low, plain / scaling.factor, blended))
        return stretched.to(torch.float32), 1.0

    def turning_pair(turns: float) -> float:  # the (fractional) dimension whose wavelength makes `turns` turns over the original context
        return dims * math.log(scaling.original / (2.0 * math.pi * turns)) / (2.0 * math.log(theta))

    low = max(math.floor(turning_pair(scaling.fast)), 0)
    high = min(math.ceil(turning_pair(scaling.slow)), dims - 1)
    ramp = ((index - low) / max(high - low, 0.001)).clamp(0.0, 1.0)
    stretched = plain / scaling.factor * ramp + plain * (1.0 - ramp)
    return stretched.to(torch.float32), 0.1 * math.log(scaling.factor) + 1.0
