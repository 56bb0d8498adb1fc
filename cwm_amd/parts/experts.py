"""Routed experts: a feed-forward of which each token uses a few."""

from __future__ import annotations

from typing import Any, Dict, Mapping

import torch

from .. import ops
from .base import FeedForward, Runtime, TensorSpec, register_part


class RoutedExperts(FeedForward):
    """z = W_router x in float32; a token's `top` experts are those with the largest z, weighted by the softmax
    over these z alone; out = sum_e weight_e * W_down,e (silu(W_gate,e x) * (W_up,e x)), no biases.

    The step's (token, expert) pairs are grouped by expert on the device (no count comes to the host), each
    group's rows padded to whole tiles, and two grouped products run over the tiles: gate/up with the
    activation in its epilogue, then down into one float32 row a pair; a last kernel adds a token's rows in the
    order of its router's choice, so a token's result does not depend on what else is in the step.
    Tensors: `router` [experts, dim] and `e<i>.gate`, `e<i>.up` [hidden, dim], `e<i>.down` [dim, hidden]."""

    replayable = True

    def __init__(self, dim: int, hidden_dim: int, n_experts: int, top: int) -> None:
        if not 1 <= top <= n_experts:
            raise ValueError(f"{top} experts a token out of {n_experts}")
        if top > ops.MAX_ROUTE_TOP or n_experts > ops.MAX_EXPERTS:
            raise ValueError(f"the routing kernels take up to {ops.MAX_ROUTE_TOP} of up to {ops.MAX_EXPERTS} experts")
        self.dim, self.hidden_dim, self.n_experts, self.top = dim, hidden_dim, n_experts, top

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {"router": TensorSpec((self.n_experts, self.dim))}
        for e in range(self.n_experts):
            specs[f"e{e}.gate"] = TensorSpec((self.hidden_dim, self.dim))
            specs[f"e{e}.up"] = TensorSpec((self.hidden_dim, self.dim))
            specs[f"e{e}.down"] = TensorSpec((self.dim, self.hidden_dim))
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.router = tensors["router"].contiguous()
        stack = lambda name: torch.stack([tensors[f"e{e}.{name}"] for e in range(self.n_experts)]).contiguous()  # noqa: E731
        self.gate, self.up, self.down = stack("gate"), stack("up"), stack("down")  # [experts, out, in]

    def forward(self, x: torch.Tensor, batch: Any) -> torch.Tensor:
        logits = ops.linear(x, self.router, None, torch.float32)
        chosen, weights = ops.route_top(logits, self.top)
        groups = ops.group_by_expert(chosen, self.n_experts)
        hidden = ops.grouped_gate_up(x, groups, self.gate, self.up)
        rows = ops.grouped_linear(hidden, groups, self.down)
        return ops.combine_routed(rows, groups, weights)  # float32 [T, dim]


register_part("feed_forward", "routed_experts", RoutedExperts)
