"""Typed configuration of the Segedra decoder.

config.json names the vocabulary and the width, the embedding's scale, one eps for every norm, the number of
residual streams (absent: a single residual with plain sums), a list of layers, and optionally a loop: a range
of layers that runs several times in a row with the same weights.  Every layer names its mixer (`type`), the
mixer's sizes (`mixer`) and its feed-forward (`mlp`, null for none), which is dense or a mixture of experts.
Strict as every configuration: an unknown key is an error that names it.
"""

from __future__ import annotations

import re
from dataclasses import dataclass
from typing import Any, List, Mapping, Optional

from .schema import ConfigError, from_dict


@dataclass(frozen=True)
class EmbeddingConfig:
    scale: float = 1.0


@dataclass(frozen=True)
class NormConfig:
    eps: float

    def __post_init__(self) -> None:
        if self.eps <= 0:
            raise ConfigError("norm.eps must be positive")


@dataclass(frozen=True)
class RotationConfig:
    base: float
    dims: int

    def __post_init__(self) -> None:
        if self.dims < 0 or self.dims % 2 != 0:
            raise ConfigError("rot.dims must be even and not negative")
        if self.base <= 0:
            raise ConfigError("rot.base must be positive")


@dataclass(frozen=True)
class MaskConfig:
    size: int  # keys a query reads, its own included

    def __post_init__(self) -> None:
        if self.size < 1:
            raise ConfigError("mask.size must be at least 1")


@dataclass(frozen=True)
class AttentionConfig:
    """`heads` query heads and `kv_heads` key/value heads; queries and keys of `dim`, values of `vdim` per head."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[RotationConfig] = None
    mask: Optional[MaskConfig] = None

    def __post_init__(self) -> None:
        if min(self.heads, self.kv_heads, self.dim, self.vdim) < 1:
            raise ConfigError("an attention mixer's sizes must be positive")
        if self.heads % self.kv_heads != 0:
            raise ConfigError(f"{self.heads} query heads do not divide into {self.kv_heads} key/value heads")
        if self.rot is not None and self.rot.dims > self.dim:
            raise ConfigError(f"rot.dims {self.rot.dims} exceeds the head's {self.dim} dimensions")


@dataclass(frozen=True)
class RouterConfig:
    experts: int
    top: int
    scale: float = 1.0

    def __post_init__(self) -> None:
        if not 1 <= self.top <= self.experts:
            raise ConfigError(f"router.top {self.top} must lie in 1..{self.experts}")


@dataclass(frozen=True)
class ExpertConfig:
    ff: int
    limit: float

    def __post_init__(self) -> None:
        if self.ff < 1 or self.limit <= 0:
            raise ConfigError("an expert needs a positive width and a positive limit")


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str
    ff: Optional[int] = None  # dense
    expert: Optional[ExpertConfig] = None  # moe
    router: Optional[RouterConfig] = None  # moe

    def __post_init__(self) -> None:
        if self.kind == "dense":
            if self.ff is None or self.ff < 1 or self.expert is not None or self.router is not None:
                raise ConfigError("a dense feed-forward names its width `ff` and nothing of experts")
        elif self.kind == "moe":
            if self.expert is None or self.router is None or self.ff is not None:
                raise ConfigError("a mixture of experts names `expert` and `router`, and no width of its own")
        else:
            raise ConfigError(f"mlp.kind {self.kind!r}: 'dense' and 'moe' are known")


MIXER_CONFIGS = {"attention": AttentionConfig}


@dataclass(frozen=True)
class LayerConfig:
    type: str
    mixer: Any
    mlp: Optional[FeedForwardConfig] = None

    def __post_init__(self) -> None:
        self.mixer_config()  # reject what does not fit now, by key

    def mixer_config(self) -> AttentionConfig:
        kind = re.sub(r"_\d+$", "", self.type)  # a numeric suffix marks another set of sizes of the same mixer
        if kind not in MIXER_CONFIGS:
            raise ConfigError(f"layer type {self.type!r}: known mixers are {', '.join(sorted(MIXER_CONFIGS))}")
        if not isinstance(self.mixer, Mapping):
            raise ConfigError(f"the sizes of mixer {self.type!r} must be an object")
        return from_dict(MIXER_CONFIGS[kind], self.mixer, path="mixer")


@dataclass(frozen=True)
class LoopConfig:
    """Layers start .. stop - 1 run `times` times in a row; each pass has a cache of its own."""

    start: int
    stop: int
    times: int

    def __post_init__(self) -> None:
        if self.start < 0 or self.stop < self.start or self.times < 1:
            raise ConfigError("loop needs 0 <= start <= stop and times >= 1")


@dataclass(frozen=True)
class SegedraConfig:
    architecture: str
    vocab: int
    width: int
    norm: NormConfig
    layers: List[LayerConfig]
    embedding: EmbeddingConfig = EmbeddingConfig()
    streams: Optional[int] = None  # None: one residual, plain sums, no connection tensors
    loop: Optional[LoopConfig] = None
    max_positions: Optional[int] = None  # not a key of the design: only cache sizing reads it when given

    def __post_init__(self) -> None:
        if self.vocab < 1 or self.width < 1:
            raise ConfigError("vocab and width must be positive")
        if not self.layers:
            raise ConfigError("a model needs at least one layer")
        if self.streams is not None and self.streams < 1:
            raise ConfigError("streams must be at least 1")
        if self.loop is not None and self.loop.stop > len(self.layers):
            raise ConfigError(f"loop.stop {self.loop.stop} exceeds the {len(self.layers)} layers")

    def layer_order(self) -> List[int]:
        """The layers in the order they run, the loop written out."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        lp = self.loop
        return list(range(lp.start)) + list(range(lp.start, lp.stop)) * lp.times + list(range(lp.stop, n))
