"""How a layer's parts are arranged."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, CacheNeed, Part, TensorSpec, prefixed, under


class Block(Part):
    """`forward(hidden, delta, batch, cell)`: `hidden` is the float32 residual
    stream [T, hidden] and `delta` what the layer before still has to add to it
    (None at the first layer).  Returns this layer's own pending delta."""

    def forward(self, hidden, delta, batch, cell) -> torch.Tensor:
        raise NotImplementedError


@dataclass(frozen=True)
class PreNormBlockSpec:
    """h += mixer(norm(h)); h += feed_forward(norm(h)).  The `*_name` fields are
    the prefixes of the sub-parts' tensors below the layer's own prefix.  A layer without a
    feed-forward has `feed_forward` None (and no norm for it)."""

    mixer_norm: Any
    mixer: Any
    feed_forward_norm: Any
    feed_forward: Any
    mixer_norm_name: str = "input_layernorm."
    mixer_name: str = "self_attn."
    feed_forward_norm_name: str = "post_attention_layernorm."
    feed_forward_name: str = "mlp."
    kind: str = "prenorm"


@BLOCKS.register("prenorm")
class PreNormBlock(Block):
    """Reference `model.py:199-201`.  Each residual add is done by the norm that
    follows it, so the stream is read and written once per sub-layer."""

    @classmethod
    def _members(cls, spec: PreNormBlockSpec):
        members = [(spec.mixer_norm_name, NORMS, spec.mixer_norm), (spec.mixer_name, MIXERS, spec.mixer)]
        if spec.feed_forward is not None:
            members.append((spec.feed_forward_norm_name, NORMS, spec.feed_forward_norm))
            members.append((spec.feed_forward_name, FEED_FORWARDS, spec.feed_forward))
        return tuple(members)

    @classmethod
    def tensors(cls, spec: PreNormBlockSpec) -> dict[str, TensorSpec]:
        found: dict[str, TensorSpec] = {}
        for name, registry, member in cls._members(spec):
            found.update(prefixed(registry.tensors(member), name))
        return found

    @classmethod
    def cache_need(cls, spec: PreNormBlockSpec) -> CacheNeed:
        return MIXERS.cache_need(spec.mixer)

    def __init__(self, spec: PreNormBlockSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        built = [
            registry.build(member, under(tensors, name), kernels)
            for name, registry, member in self._members(spec)
        ]
        self.mixer_norm, self.mixer = built[:2]
        self.feed_forward_norm, self.feed_forward = built[2:] if len(built) > 2 else (None, None)
        self.replayable = all(part.replayable for part in built)

    def forward(self, hidden, delta, batch, cell) -> torch.Tensor:
        normed = self.mixer_norm.forward(hidden, delta)
        mixed = self.mixer.forward(normed, batch, cell)
        if self.feed_forward is None:
            return mixed
        normed = self.feed_forward_norm.forward(hidden, mixed)
        return self.feed_forward.forward(normed, batch)


@dataclass(frozen=True)
class OutputNormBlockSpec:
    """h += norm(mixer(h)); h += norm(feed_forward(h)): the sublayers read the stream itself, and the norms act on
    what they return.  Fields as in `PreNormBlockSpec`."""

    mixer_norm: Any
    mixer: Any
    feed_forward_norm: Any
    feed_forward: Any
    mixer_norm_name: str = "norm1."
    mixer_name: str = "mix."
    feed_forward_norm_name: str = "norm2."
    feed_forward_name: str = "mlp."
    kind: str = "outnorm"


@BLOCKS.register("outnorm")
class OutputNormBlock(PreNormBlock):
    """The stream is float32; a sublayer reads it rounded to the run dtype, and the kernel that adds a normed result to
    the stream also writes that rounded copy for the next sublayer (of this layer or of the next one, which finds it
    on the step).  Nothing is left pending: the block returns None."""

    def forward(self, hidden, delta, batch, cell):
        kept = batch.computed.get("stream rows")
        if delta is None and kept is not None and kept[0] is hidden:
            rows = kept[1]
        else:
            rows = self.kernels.stream_rows(hidden, delta)
        rows = self.mixer_norm.add_normed(hidden, self.mixer.forward(rows, batch, cell))
        if self.feed_forward is not None:
            rows = self.feed_forward_norm.add_normed(hidden, self.feed_forward.forward(rows, batch))
        batch.computed["stream rows"] = (hidden, rows)
        return None


@dataclass
class PendingNormed:
    """What a sublayer leaves for the stream when its result is normed before it is added: `hidden += update *
    rsqrt(mean(update^2) + eps) * weight` is still to do (`update` float32 rows, or partial sums of them).  The next
    block of the same kind does it in the kernel that norms the stream for its mixer; anyone else calls `settle`."""

    update: torch.Tensor
    weight: torch.Tensor
    eps: float
    kernels: Any

    def settle(self, hidden: torch.Tensor) -> None:
        self.kernels.add_normed(hidden, self.update, self.weight, self.eps)
        return None


@dataclass(frozen=True)
class SandwichBlockSpec:
    """h += scale1 * norm1b(mixer(norm1(h))); h += scale2 * norm2b(feed_forward(norm2(h))): a norm before and one behind
    every sublayer, and a learned vector (`*_scale_name`, as long as a row; None: none) on what is added.  A layer
    without a feed-forward has `feed_forward` None.  The `*_name` fields are the prefixes (the scales' the names) of
    the members' tensors below the layer's own prefix."""

    mixer_norm: Any
    mixer: Any
    mixer_out_norm: Any
    feed_forward_norm: Any
    feed_forward: Any
    feed_forward_out_norm: Any
    mixer_norm_name: str = "norm1."
    mixer_name: str = "mix."
    mixer_out_norm_name: str = "norm1b."
    feed_forward_norm_name: str = "norm2."
    feed_forward_name: str = "mlp."
    feed_forward_out_norm_name: str = "norm2b."
    mixer_scale_name: str | None = "ls1"
    feed_forward_scale_name: str | None = "ls2"
    kind: str = "sandwich"


@BLOCKS.register("sandwich")
class SandwichBlock(Block):
    """The norms are RMS norms with a weight.  The vector on a sublayer's result is multiplied into the weight of the
    norm behind the sublayer when the block is built (float32), so it costs nothing in a step.  The norm behind a
    sublayer, the add and the norm before the next sublayer are one kernel: the stream is read and written once a
    sublayer.  What the last sublayer leaves is handed on as a `PendingNormed`."""

    accepts_pending_normed = True

    @classmethod
    def _members(cls, spec: SandwichBlockSpec):
        members = [
            (spec.mixer_norm_name, NORMS, spec.mixer_norm), (spec.mixer_name, MIXERS, spec.mixer),
            (spec.mixer_out_norm_name, NORMS, spec.mixer_out_norm),
        ]
        if spec.feed_forward is not None:
            members += [
                (spec.feed_forward_norm_name, NORMS, spec.feed_forward_norm), (spec.feed_forward_name, FEED_FORWARDS, spec.feed_forward),
                (spec.feed_forward_out_norm_name, NORMS, spec.feed_forward_out_norm),
            ]
        return tuple(members)

    @classmethod
    def tensors(cls, spec: SandwichBlockSpec) -> dict[str, TensorSpec]:
        found: dict[str, TensorSpec] = {}
        for name, registry, member in cls._members(spec):
            found.update(prefixed(registry.tensors(member), name))
        if spec.mixer_scale_name is not None:
            found[spec.mixer_scale_name] = TensorSpec((spec.mixer_out_norm.size,), role="norm")
        if spec.feed_forward is not None and spec.feed_forward_scale_name is not None:
            found[spec.feed_forward_scale_name] = TensorSpec((spec.feed_forward_out_norm.size,), role="norm")
        return found

    @classmethod
    def cache_need(cls, spec: SandwichBlockSpec) -> CacheNeed:
        return MIXERS.cache_need(spec.mixer)

    def __init__(self, spec: SandwichBlockSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        built = [registry.build(member, under(tensors, name), kernels) for name, registry, member in self._members(spec)]
        for norm in (built[0], built[2], *(built[3::2])):
            if not hasattr(norm, "weight") or hasattr(norm, "bias"):
                raise ValueError("sandwich block: its norms are RMS norms with a weight")
        self.mixer_norm, self.mixer = built[0], built[1]

        def scaled(norm, name):
            weight = norm.weight.float()
            return (weight * tensors[name].float() if name is not None else weight).contiguous()

        self.mixer_out = scaled(built[2], spec.mixer_scale_name)
        self.mixer_out_eps = spec.mixer_out_norm.eps
        self.feed_forward_norm = self.feed_forward = self.feed_forward_out = None
        if spec.feed_forward is not None:
            self.feed_forward_norm, self.feed_forward = built[3], built[4]
            self.feed_forward_out = scaled(built[5], spec.feed_forward_scale_name)
            self.feed_forward_out_eps = spec.feed_forward_out_norm.eps
        self.replayable = all(part.replayable for part in built)

    def forward(self, hidden, delta, batch, cell):
        kernels = self.kernels
        if isinstance(delta, PendingNormed):
            normed = kernels.add_normed_norm(hidden, delta.update, delta.weight, delta.eps, self.mixer_norm.weight, self.mixer_norm.spec.eps)
        else:
            normed = self.mixer_norm.forward(hidden, delta)
        mixed = self.mixer.forward(normed, batch, cell)
        if self.feed_forward is None:
            return PendingNormed(mixed, self.mixer_out, self.mixer_out_eps, kernels)
        normed = kernels.add_normed_norm(
            hidden, mixed, self.mixer_out, self.mixer_out_eps, self.feed_forward_norm.weight, self.feed_forward_norm.spec.eps
        )
        fed = self.feed_forward.forward(normed, batch)
        return PendingNormed(fed, self.feed_forward_out, self.feed_forward_out_eps, kernels)
