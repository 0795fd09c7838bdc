"""A feed-forward of many small experts, a few of which each token uses, and an optional shared one."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .base import FEED_FORWARDS, TensorSpec
from .feed_forward import FeedForward


@dataclass(frozen=True)
class RoutedExpertsSpec:
    """`num_experts` experts down(act(up x)) of width `expert_size` (with `gated`: down(act(gate x) * up x)), `top`
    of them a token.  The router's scores are squashed by `scoring` ("sigmoid", or "softmax" over all experts); an
    expert is chosen by score + correction (`correction` False: by score alone, and no such tensor) among the
    experts of the `keep_groups` best of `groups` equal groups of neighbours (a group's score is its largest), and
    weighted by its score times `route_scale`; with `renormalise` the chosen scores are divided by their sum (+ 1e-20)
    first.  `shared_size` (None: none) is the width of an expert that every token uses, of the same form, scaled by
    sigmoid of a gate of its own (`shared_gate` False: added as it is).  `router_bias`: the router's logits have a bias
    (`router.b`), part of the float32 product.  `limit`: of the activation "limited_swish" (g = min(gate, limit), u =
    clamp(up, -limit, limit), g sigmoid(1.702 g) (u + 1)).  A softmax over the chosen logits alone is `scoring`
    "softmax" with `renormalise`: the sum over all experts cancels."""

    hidden_size: int
    num_experts: int
    top: int
    expert_size: int
    route_scale: float
    activation: str = "gelu"
    scoring: str = "sigmoid"
    shared_size: int | None = None
    shared_activation: str = "gelu"
    gated: bool = False
    correction: bool = True
    groups: int = 1
    keep_groups: int = 1
    renormalise: bool = False
    shared_gate: bool = True
    router_bias: bool = False
    limit: float | None = None
    kind: str = "routed_experts"


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    """z = W_router x in float32, s = squash(z); the `top` largest of s + correction choose the experts;
    y = sum over the chosen e of route_scale s_e down_e(act(up_e x)) (+ sigmoid(W_sg x) shared(x)).
    The choice is made on the device: the tokens' rows are sorted by expert there and the experts run as one
    grouped product, so a step is the same launches whatever the data."""

    @classmethod
    def tensors(cls, spec: RoutedExpertsSpec) -> dict[str, TensorSpec]:
        found = {"router": TensorSpec((spec.num_experts, spec.hidden_size))}
        if spec.router_bias:
            found["router.b"] = TensorSpec((spec.num_experts,), role="bias")
        if spec.correction:
            found["correction"] = TensorSpec((spec.num_experts,), role="bias")
        for index in range(spec.num_experts):
            if spec.gated:
                found[f"e{index}.gate"] = TensorSpec((spec.expert_size, spec.hidden_size))
            found[f"e{index}.up"] = TensorSpec((spec.expert_size, spec.hidden_size))
            found[f"e{index}.down"] = TensorSpec((spec.hidden_size, spec.expert_size))
        if spec.shared_size is not None:
            if spec.gated:
                found["shared.gate"] = TensorSpec((spec.shared_size, spec.hidden_size))
            found["shared.up"] = TensorSpec((spec.shared_size, spec.hidden_size))
            found["shared.down"] = TensorSpec((spec.hidden_size, spec.shared_size))
            if spec.shared_gate:
                found["shared.sg"] = TensorSpec((1, spec.hidden_size))
        return found

    def __init__(self, spec: RoutedExpertsSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        if not 0 < spec.top <= spec.num_experts:
            raise ValueError("routed experts: a token uses between one and all of the experts")
        if spec.num_experts % spec.groups or not 0 < spec.keep_groups <= spec.groups or spec.top > spec.keep_groups * (spec.num_experts // spec.groups):
            raise ValueError("routed experts: equal groups, between one and all of them kept, with room for a token's experts")
        shared = spec.shared_size is not None
        # the shared expert's gate is one more row of the router's product
        gate_row = [tensors["shared.sg"]] if shared and spec.shared_gate else []
        biases = None
        if spec.router_bias:
            biases = [tensors["router.b"]] + [torch.zeros((1,), dtype=tensors["router.b"].dtype, device=tensors["router.b"].device) for _ in gate_row]
        self.router = kernels.prepare_linear([tensors["router"]] + gate_row, biases)
        self.correction = kernels.to_device(tensors["correction"].float().contiguous()) if spec.correction else None
        self.experts = kernels.prepare_experts(
            [tensors[f"e{index}.up"] for index in range(spec.num_experts)],
            [tensors[f"e{index}.down"] for index in range(spec.num_experts)],
            spec.activation,
            gates=[tensors[f"e{index}.gate"] for index in range(spec.num_experts)] if spec.gated else None,
            **({"limit": spec.limit} if spec.limit is not None else {}),
        )
        self.shared_up = self.shared_down = None
        if shared:
            if spec.gated:
                self.shared_up = kernels.prepare_gated_linear(tensors["shared.gate"], tensors["shared.up"], spec.shared_activation)
            else:
                self.shared_up = kernels.prepare_linear([tensors["shared.up"]], None)
            self.shared_down = kernels.prepare_linear([tensors["shared.down"]], None)

    def forward(self, x: torch.Tensor, batch) -> torch.Tensor:
        kernels, spec = self.kernels, self.spec
        scores = kernels.linear(x, self.router, out_dtype=torch.float32)  # [T, experts (+ 1)]
        chosen, weights = kernels.route(
            scores, spec.num_experts, self.correction, spec.top, spec.route_scale, spec.scoring,
            groups=spec.groups, keep_groups=spec.keep_groups, renormalise=spec.renormalise,
        )
        if self.shared_up is None:
            return kernels.expert_feed_forward(x, self.experts, chosen, weights)  # float32 [T, hidden]
        if spec.gated:
            inner = kernels.gated_linear(x, self.shared_up)
        else:
            inner = kernels.activate(kernels.linear(x, self.shared_up), spec.shared_activation)
        shared = kernels.linear(inner, self.shared_down, out_dtype=torch.float32)
        # the kernel that adds a token's experts up adds the (gated) shared expert too
        if not spec.shared_gate:
            return kernels.expert_feed_forward(x, self.experts, chosen, weights, shared=shared)
        return kernels.expert_feed_forward(x, self.experts, chosen, weights, shared=shared, gates=scores, gate_column=spec.num_experts)
