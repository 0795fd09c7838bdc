"""Several copies of the residual stream that the sublayers read from and write to through learned weights
(hyper-connections): a sublayer reads one weighted sum of the copies, and its result goes to every copy with a
weight of its own while the copies themselves are mixed by a small matrix."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

from .base import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, STREAM_PARTS, CacheNeed, Part, TensorSpec, prefixed, under
from .block import Block


@dataclass
class PendingWrite:
    """What a sublayer still has to do to the copies: x_t <- sum_s mix[s, t] x_s + out[t] * result.  `result` is
    float32 [T, hidden] or partial sums [parts, T, hidden]; `mix` float32 [copies, copies] (from, to), `out`
    float32 [copies].  The kernel that reads the copies for the next sublayer does it on the way."""

    result: torch.Tensor
    mix: torch.Tensor
    out: torch.Tensor

    def applied(self, streams: torch.Tensor) -> torch.Tensor:
        """The copies [T, copies * hidden] as they are after this write (for tests and debugging: plain torch)."""
        copies = self.out.shape[0]
        result = self.result if self.result.ndim == 2 else self.result.sum(0)
        old = streams.view(streams.shape[0], copies, -1)
        new = torch.einsum("st,nsh->nth", self.mix.to(old.device), old) + self.out.to(old.device)[None, :, None] * result[:, None, :]
        return new.reshape(streams.shape)


@dataclass(frozen=True)
class StreamCopiesSpec:
    """The embedded rows times `scale`, `copies` times side by side: [T, hidden] -> [T, copies * hidden]."""

    copies: int
    scale: float = 1.0
    kind: str = "stream_copies"


@STREAM_PARTS.register("stream_copies")
class StreamCopies(Part):
    def __init__(self, spec: StreamCopiesSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        if spec.copies < 1:
            raise ValueError("stream copies: at least one copy")

    def forward(self, hidden: torch.Tensor, batch) -> torch.Tensor:
        return self.kernels.stream_copies(hidden, self.spec.copies, self.spec.scale)


@dataclass(frozen=True)
class StreamNormSpec:
    """RMS norm of a weighted sum of `copies` copies of the stream.  With `read_name` None every copy weighs one
    (the sum of the copies: what stands before a model's head)."""

    size: int
    eps: float
    copies: int
    weight_name: str = "weight"
    read_name: str | None = None
    kind: str = "stream_rmsnorm"


@NORMS.register("stream_rmsnorm")
class StreamNorm(Part):
    """u = sum_s read[s] x_s; y = u * rsqrt(mean(u^2) + eps) * weight, float32, with the write that the sublayer
    before left pending done in the same kernel.  The read weights may be handed over by a block that owns them."""

    @classmethod
    def tensors(cls, spec: StreamNormSpec) -> dict[str, TensorSpec]:
        found = {spec.weight_name: TensorSpec((spec.size,), role="norm")}
        if spec.read_name is not None:
            found[spec.read_name] = TensorSpec((spec.copies,), role="norm")
        return found

    def __init__(self, spec: StreamNormSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        self.weight = tensors[spec.weight_name]
        read = tensors[spec.read_name].float() if spec.read_name is not None else torch.ones(spec.copies)
        self.read = kernels.to_device(read.contiguous())

    def forward(self, streams: torch.Tensor, pending: PendingWrite | None) -> torch.Tensor:
        """Does the pending write (in place) and returns the normed rows in the run dtype."""
        return self.kernels.stream_norm(streams, pending, self.read, self.weight, self.spec.eps)

    def forward_rows(self, streams: torch.Tensor, pending: PendingWrite | None, rows: torch.Tensor) -> torch.Tensor:
        """The same for the token rows `rows` alone, the copies left as they are (after the last layer)."""
        return self.kernels.stream_norm(streams, pending, self.read, self.weight, self.spec.eps, rows=rows)


@dataclass(frozen=True)
class HyperBlockSpec:
    """For sublayer q (mixer, feed-forward): u = sum_s in_q[s] x_s; y = sublayer(norm_q(u)); then, all copies at
    once from the old ones, x_t <- sum_s mix_q[s, t] x_s + out_q[t] y.  A layer without a feed-forward has
    `feed_forward` None.  The `*_name` fields are the prefixes below the layer's own prefix; `mixer_links` and
    `feed_forward_links` those of the tensors `in` [copies], `out` [copies] and `mix` [copies, copies]."""

    copies: int
    mixer_norm: Any
    mixer: Any
    feed_forward_norm: Any
    feed_forward: Any
    mixer_norm_name: str = "norm1"
    mixer_name: str = "mix."
    feed_forward_norm_name: str = "norm2"
    feed_forward_name: str = "mlp."
    mixer_links: str = "hc1."
    feed_forward_links: str = "hc2."
    learned_links: bool = True  # False: no such tensors; every weight is one (one copy: the plain residual sum x <- x + y)
    kind: str = "hyper"


def _links(copies: int) -> dict[str, TensorSpec]:
    return {"in": TensorSpec((copies,), role="norm"), "out": TensorSpec((copies,), role="norm"), "mix": TensorSpec((copies, copies), role="bias")}


@BLOCKS.register("hyper")
class HyperBlock(Block):
    """`hidden` is the copies side by side, float32 [T, copies * hidden]; what a block leaves pending is a
    `PendingWrite`, done by whoever reads the copies next (the next block's first norm, or the model's last)."""

    @classmethod
    def _members(cls, spec: HyperBlockSpec):
        members = [(spec.mixer_norm_name, NORMS, spec.mixer_norm), (spec.mixer_name, MIXERS, spec.mixer)]
        if spec.feed_forward is not None:
            members.append((spec.feed_forward_norm_name, NORMS, spec.feed_forward_norm))
            members.append((spec.feed_forward_name, FEED_FORWARDS, spec.feed_forward))
        return tuple(members)

    @classmethod
    def tensors(cls, spec: HyperBlockSpec) -> dict[str, TensorSpec]:
        found: dict[str, TensorSpec] = {}
        for name, registry, member in cls._members(spec):
            found.update(prefixed(registry.tensors(member), name))
        if spec.learned_links:
            found.update(prefixed(_links(spec.copies), spec.mixer_links))
            if spec.feed_forward is not None:
                found.update(prefixed(_links(spec.copies), spec.feed_forward_links))
        return found

    @classmethod
    def cache_need(cls, spec: HyperBlockSpec) -> CacheNeed:
        return MIXERS.cache_need(spec.mixer)

    def __init__(self, spec: HyperBlockSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        built = [registry.build(member, under(tensors, name), kernels) for name, registry, member in self._members(spec)]
        self.mixer_norm, self.mixer = built[:2]
        self.feed_forward_norm, self.feed_forward = built[2:] if len(built) > 2 else (None, None)
        self.replayable = all(part.replayable for part in built)

        if not spec.learned_links and spec.copies != 1:
            raise ValueError("hyper block: several copies of the stream need their links")

        def links(prefix: str):
            if not spec.learned_links:
                return tuple(kernels.to_device(torch.ones(shape)) for shape in ((1,), (1, 1), (1,)))
            own = under(tensors, prefix)
            return tuple(kernels.to_device(own[name].float().contiguous()) for name in ("in", "mix", "out"))

        self.mixer_read, self.mixer_mix, self.mixer_out = links(spec.mixer_links)
        if self.feed_forward is not None:
            self.feed_read, self.feed_mix, self.feed_out = links(spec.feed_forward_links)

    def forward(self, hidden, delta, batch, cell) -> PendingWrite:
        kernels, eps = self.kernels, self.mixer_norm.spec.eps
        normed = kernels.stream_norm(hidden, delta, self.mixer_read, self.mixer_norm.weight, eps)
        pending = PendingWrite(self.mixer.forward(normed, batch, cell), self.mixer_mix, self.mixer_out)
        if self.feed_forward is None:
            return pending
        normed = kernels.stream_norm(hidden, pending, self.feed_read, self.feed_forward_norm.weight, self.feed_forward_norm.spec.eps)
        return PendingWrite(self.feed_forward.forward(normed, batch), self.feed_mix, self.feed_out)
