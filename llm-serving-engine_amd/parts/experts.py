"""A feed-forward of many small experts, a few of which each token uses, and an optional shared one."""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .base import FEED_FORWARDS, TensorSpec
from .feed_forward import FeedForward


@dataclass(frozen=True)
class RoutedExpertsSpec:
    """`num_experts` experts down(act(up x)) of width `expert_size`, `top` of them a token.  The router's
    scores are squashed by `scoring` ("sigmoid"); an expert is chosen by score + correction and weighted by
    its score times `route_scale`, not renormalised.  `shared_size` (None: none) is the width of an expert
    that every token uses, scaled by sigmoid of a gate of its own."""

    hidden_size: int
    num_experts: int
    top: int
    expert_size: int
    route_scale: float
    activation: str = "gelu"
    scoring: str = "sigmoid"
    shared_size: int | None = None
    shared_activation: str = "gelu"
    kind: str = "routed_experts"


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    """z = W_router x in float32, s = squash(z); the `top` largest of s + correction choose the experts;
    y = sum over the chosen e of route_scale s_e down_e(act(up_e x)) (+ sigmoid(W_sg x) shared(x)).
    The choice is made on the device: the tokens' rows are sorted by expert there and the experts run as one
    grouped product, so a step is the same launches whatever the data."""

    @classmethod
    def tensors(cls, spec: RoutedExpertsSpec) -> dict[str, TensorSpec]:
        found = {"router": TensorSpec((spec.num_experts, spec.hidden_size)), "correction": TensorSpec((spec.num_experts,), role="bias")}
        for index in range(spec.num_experts):
            found[f"e{index}.up"] = TensorSpec((spec.expert_size, spec.hidden_size))
            found[f"e{index}.down"] = TensorSpec((spec.hidden_size, spec.expert_size))
        if spec.shared_size is not None:
            found["shared.up"] = TensorSpec((spec.shared_size, spec.hidden_size))
            found["shared.down"] = TensorSpec((spec.hidden_size, spec.shared_size))
            found["shared.sg"] = TensorSpec((1, spec.hidden_size))
        return found

    def __init__(self, spec: RoutedExpertsSpec, tensors, kernels) -> None:
        super().__init__(spec, tensors, kernels)
        if not 0 < spec.top <= spec.num_experts:
            raise ValueError("routed experts: a token uses between one and all of the experts")
        shared = spec.shared_size is not None
        # the shared expert's gate is one more row of the router's product
        self.router = kernels.prepare_linear([tensors["router"]] + ([tensors["shared.sg"]] if shared else []), None)
        self.correction = kernels.to_device(tensors["correction"].float().contiguous())
        self.experts = kernels.prepare_experts(
            [tensors[f"e{index}.up"] for index in range(spec.num_experts)],
            [tensors[f"e{index}.down"] for index in range(spec.num_experts)],
            spec.activation,
        )
        self.shared_up = kernels.prepare_linear([tensors["shared.up"]], None) if shared else None
        self.shared_down = kernels.prepare_linear([tensors["shared.down"]], None) if shared else None

    def forward(self, x: torch.Tensor, batch) -> torch.Tensor:
        kernels, spec = self.kernels, self.spec
        scores = kernels.linear(x, self.router, out_dtype=torch.float32)  # [T, experts (+ 1)]
        chosen, weights = kernels.route(scores, spec.num_experts, self.correction, spec.top, spec.route_scale, spec.scoring)
        if self.shared_up is None:
            return kernels.expert_feed_forward(x, self.experts, chosen, weights)  # float32 [T, hidden]
        inner = kernels.activate(kernels.linear(x, self.shared_up), spec.shared_activation)
        shared = kernels.linear(inner, self.shared_down, out_dtype=torch.float32)
        # the kernel that adds a token's experts up adds the gated shared expert too
        return kernels.expert_feed_forward(x, self.experts, chosen, weights, shared=shared, gates=scores, gate_column=spec.num_experts)
