"""Several mixers side by side that read the same rows; their results are added with a weight each."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

from .attention import Mixer
from .base import MIXERS, CacheNeed, TensorSpec, prefixed, under


@dataclass(frozen=True)
class ParallelMixersSpec:
    """`members`: (prefix of the member's tensors below the part's own, the member's spec, its weight in the sum)."""

    members: tuple[tuple[str, Any, float], ...]
    kind: str = "parallel"


@MIXERS.register("parallel")
class ParallelMixers(Mixer):
    """result = sum_m weight_m mixer_m(x), float32.  What the members keep in the cache is kept side by side under
    `<member's prefix><name>` (a member with one need: under its prefix alone)."""

    @classmethod
    def tensors(cls, spec: ParallelMixersSpec) -> dict[str, TensorSpec]:
        found: dict[str, TensorSpec] = {}
        for prefix, member, _ in spec.members:
            found.update(prefixed(MIXERS.tensors(member), prefix))
        return found

    @classmethod
    def cache_need(cls, spec: ParallelMixersSpec) -> dict[str, CacheNeed] | None:
        need: dict[str, CacheNeed] = {}
        for prefix, member, _ in spec.members:
            own = MIXERS.cache_need(member)
            if isinstance(own, dict):
                need.update(prefixed(own, prefix))
            elif own is not None:
                need[prefix] = own
        return need or None

    def __init__(self, spec: ParallelMixersSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        if not spec.members:
            raise ValueError("parallel mixers: no members")
        self.members = [MIXERS.build(member, under(tensors, prefix), kernels) for prefix, member, _ in spec.members]
        self.replayable = all(member.replayable for member in self.members)

    def forward(self, x: torch.Tensor, batch, cell) -> torch.Tensor:
        results = []
        for (prefix, member_spec, weight), member in zip(self.spec.members, self.members):
            own = MIXERS.cache_need(member_spec)
            if isinstance(own, dict):
                member_cell = under(cell, prefix)
            else:
                member_cell = cell[prefix] if own is not None else None
            results.append((member.forward(x, batch, member_cell), float(weight)))
        total, weight = results[0]
        for other, other_weight in results[1:]:
            total, weight = self.kernels.add_scaled(total, weight, other, other_weight), 1.0
        if weight != 1.0:  # (one member alone)
            total = self.kernels.add_scaled(total, weight, None, 0.0)
        return total
