"""Selective state-space mixer (the Mamba-2 recurrence) with a per-request state."""

from __future__ import annotations

from typing import Any, Dict, Mapping

import torch

from .. import ops
from .base import Mixer, PartChoice, Runtime, StateSpec, TensorSpec, register_part
from .linear import LinearWeights


class SelectiveStateSpace(Mixer):
    """u = W_in s = [z | x | B | C | dt] with inner = heads * head_dim channels of z and x, groups * state of B
    and C, one dt a head.  (x, B, C) pass a causal convolution per channel (`taps` wide, bias) and SiLU;
    dt <- softplus(dt + dt_bias).  Per head h with its group g = h // (heads / groups), the state S (state x
    head_dim, float32) moves as
        S_t = exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T,      y_t = S_t^T C_t + D_h x_t,
    then out = W_o norm(y * silu(z)) with a group norm of `norm_groups` parts.  The recurrence, its step sizes
    and decays and the gated norm run in float32 whatever the activation type.

    A request's state is one float32 row: S of every head (in the order the scan kernel holds it), then the last
    taps - 1 inputs of the convolution (oldest first), so a portion of a prompt goes on where the step before stopped."""

    replayable = True

    def __init__(self, dim: int, heads: int, head_dim: int, state: int, groups: int, norm_groups: int, taps: int, eps: float) -> None:
        if heads % groups != 0:
            raise ValueError(f"{heads} heads do not divide into {groups} groups")
        if not 1 <= taps <= ops.MAX_CONV_TAPS:
            raise ValueError(f"a convolution of {taps} taps is outside 1..{ops.MAX_CONV_TAPS}, what the kernel takes")
        if state > ops.MAX_SSM_STATE:
            raise ValueError(f"a state of {state} rows is more than the {ops.MAX_SSM_STATE} the scan kernel takes")
        self.dim, self.heads, self.head_dim, self.state, self.groups, self.taps = dim, heads, head_dim, state, groups, taps
        self.inner = heads * head_dim
        self.channels = self.inner + 2 * groups * state  # what the convolution sees
        self.norm = PartChoice("group_rmsnorm", {"dim": self.inner, "eps": eps, "groups": norm_groups, "tensor": "norm"}).build("norm")
        self.ssm_elems = ops.scan_state_elems(heads, head_dim, state)  # in the scan kernel's own order and padding
        self.state_elems = -(-(self.ssm_elems + (taps - 1) * self.channels) // 4) * 4

    def cache_spec(self) -> StateSpec:
        return StateSpec((self.state_elems,), torch.float32)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {
            "in": TensorSpec((2 * self.inner + 2 * self.groups * self.state + self.heads, self.dim)),
            "conv": TensorSpec((self.channels, self.taps)),
            "conv.b": TensorSpec((self.channels,)),
            "dt_bias": TensorSpec((self.heads,)),
            "A_log": TensorSpec((self.heads,)),
            "D": TensorSpec((self.heads,)),
            **self.norm.tensor_specs(),
            "o": TensorSpec((self.dim, self.inner)),
        }

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.norm.bind({"norm": tensors["norm"]}, runtime)
        self.w_in = LinearWeights(tensors["in"], stream_copy=runtime.stream_copies)
        self.w_out = LinearWeights(tensors["o"], stream_copy=runtime.stream_copies)
        # everything that enters the recurrence is kept in float32 (exact from a 16-bit file)
        self.conv_w = tensors["conv"].float().contiguous()
        self.conv_w_by_tap = self.conv_w.t().contiguous()  # [taps, channels]: what portions of a prompt read
        self.conv_b = tensors["conv.b"].float().contiguous()
        self.dt_bias = tensors["dt_bias"].float().contiguous()
        self.a_log = tensors["A_log"].float().contiguous()
        self.d_skip = tensors["D"].float().contiguous()

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        if not write_cache:
            raise ValueError("a state-space mixer cannot read another layer's state")
        u = self.w_in(x)
        inner = self.inner
        z = u[:, :inner]
        xbc = ops.causal_conv_silu(
            u[:, inner : inner + self.channels], self.conv_w, self.conv_b, cache.state, self.ssm_elems, batch, self.conv_w_by_tap,
        )
        y = ops.selective_scan(
            xbc, u[:, inner + self.channels :], self.dt_bias, self.a_log, self.d_skip, cache.state, batch,
            self.heads, self.head_dim, self.state, self.groups,
        )
        return self.w_out(self.norm.gated(y, z), partials_ok=True)


register_part("mixer", "selective_state_space", SelectiveStateSpace)
