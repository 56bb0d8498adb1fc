"""Typed configuration of the Lapevik decoder.

config.json names the model's width and vocabulary, one norm rule for the whole model and a list of layers;
every layer names its mixer (`type`), the mixer's sizes (`mixer`) and its feed-forward (`mlp`, null for none).
A mixer's sizes depend on its kind, so `mixer` is kept as the dictionary it is and turned into the kind's own
dataclass by `LayerConfig.mixer_config()`, with the same strictness as every other key.  A type that ends in
`_<number>` is the kind before the suffix with another set of sizes.
"""

from __future__ import annotations

import re
from dataclasses import dataclass
from typing import Any, List, Mapping, Optional, Union

from .schema import ConfigError, from_dict


@dataclass(frozen=True)
class NormConfig:
    eps: float
    groups: int = 1

    def __post_init__(self) -> None:
        if self.groups < 1:
            raise ConfigError("norm.groups must be at least 1")


@dataclass(frozen=True)
class RotationConfig:
    base: float
    dims: int

    def __post_init__(self) -> None:
        if self.dims < 0 or self.dims % 2 != 0:
            raise ConfigError("rot.dims must be even")


@dataclass(frozen=True)
class StateSpaceConfig:
    """Sizes of a selective state-space mixer: `heads` of `vdim` channels, a state of `state` rows per head,
    `groups` sets of input and output projections of the state shared by heads / groups heads each, a causal
    convolution of `conv` taps, and a gated norm in `norm_groups` parts."""

    heads: int
    vdim: int
    state: int
    groups: int = 1
    norm_groups: int = 1
    conv: int = 4

    def __post_init__(self) -> None:
        if min(self.heads, self.vdim, self.state, self.groups, self.norm_groups, self.conv) < 1:
            raise ConfigError("a state-space mixer's sizes must be positive")
        if self.heads % self.groups != 0:
            raise ConfigError(f"{self.heads} heads do not divide into {self.groups} groups")
        if (self.heads * self.vdim) % self.norm_groups != 0:
            raise ConfigError(f"{self.heads * self.vdim} channels do not divide into {self.norm_groups} norm groups")


@dataclass(frozen=True)
class LatentAttentionConfig:
    """Sizes of attention through a latent: `heads` heads with `dim` unrotated and `rot_dim` rotated query/key
    dimensions and values of `vdim`; queries come from a latent of `q_rank`, keys and values from one of `kv_rank`."""

    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: RotationConfig

    def __post_init__(self) -> None:
        if min(self.heads, self.dim, self.vdim, self.kv_rank, self.q_rank) < 1 or self.rot_dim < 0:
            raise ConfigError("a latent attention's sizes must be positive")
        if self.rot.dims > self.rot_dim:
            raise ConfigError(f"rot.dims {self.rot.dims} exceeds rot_dim {self.rot_dim}")


@dataclass(frozen=True)
class RouterConfig:
    experts: int
    top: int

    def __post_init__(self) -> None:
        if not 1 <= self.top <= self.experts:
            raise ConfigError(f"router.top {self.top} must lie in 1..{self.experts}")


@dataclass(frozen=True)
class ExpertConfig:
    ff: int


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str
    expert: ExpertConfig
    router: RouterConfig

    def __post_init__(self) -> None:
        if self.kind != "moe":
            raise ConfigError(f"mlp.kind {self.kind!r}: 'moe' is the feed-forward of this architecture")


MIXER_CONFIGS = {"mamba2": StateSpaceConfig, "latent_attention": LatentAttentionConfig}


def mixer_kind(layer_type: str) -> str:
    """'mamba2_2' -> 'mamba2': a numeric suffix marks another set of sizes of the same mixer."""
    return re.sub(r"_\d+$", "", layer_type)


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: Any
    mlp: Optional[FeedForwardConfig] = None

    def __post_init__(self) -> None:
        self.mixer_config()  # reject what does not fit now, by key

    def mixer_config(self) -> Union[StateSpaceConfig, LatentAttentionConfig]:
        kind = mixer_kind(self.type)
        if kind not in MIXER_CONFIGS:
            raise ConfigError(f"layer type {self.type!r}: known mixers are {', '.join(sorted(MIXER_CONFIGS))}")
        if not isinstance(self.mixer, Mapping):
            raise ConfigError(f"the sizes of mixer {self.type!r} must be an object")
        return from_dict(MIXER_CONFIGS[kind], self.mixer, path="mixer")


@dataclass(frozen=True)
class LapevikConfig:
    architecture: str
    vocab: int
    width: int
    norm: NormConfig
    layers: List[LayerConfig]
    max_positions: Optional[int] = None  # not a key of the design: only cache sizing reads it when given

    def __post_init__(self) -> None:
        if self.vocab < 1 or self.width < 1:
            raise ConfigError("vocab and width must be positive")
        if self.width % self.norm.groups != 0:
            raise ConfigError(f"width {self.width} does not divide into {self.norm.groups} norm groups")
        if not self.layers:
            raise ConfigError("a model needs at least one layer")
