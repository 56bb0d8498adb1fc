"""Token shift: a mixer's input blended with the previous token's."""

from __future__ import annotations

from typing import Any, Dict, Mapping

import torch

from .. import ops
from .base import Mixer, Runtime, StateSpec, TensorSpec, register_part


class TokenShift(Mixer):
    """s_t = h_t + (h_(t-1) - h_t) * mu, element by element, with h_(-1) = 0; float32 arithmetic on the float32
    stream, the result in the activation type.  The last h of a sequence is its state (float32 [dim]), so a
    portion's first token finds what the step before left.  `tensor`: local name of mu."""

    replayable = True

    def __init__(self, dim: int, tensor: str = "weight") -> None:
        self.dim = dim
        self.tensor = tensor

    def cache_spec(self) -> StateSpec:
        return StateSpec((self.dim,), torch.float32)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.tensor: TensorSpec((self.dim,), init="normal", precision="stored")}

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.mu = tensors[self.tensor].float().contiguous()

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        return ops.token_shift(x, self.mu, cache.state, batch, self.runtime.act_dtype, write_state=write_cache)


register_part("mixer", "token_shift", TokenShift)
