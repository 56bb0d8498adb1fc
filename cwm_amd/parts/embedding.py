"""The parts at the two ends of a model: the token embedding and the output head."""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from .. import ops
from .base import Embedding, Head, PartChoice, Runtime, TensorSpec, register_part
from .linear import LinearWeights


class TokenEmbedding(Embedding):
    """h = scale * table[tokens], as the float32 residual stream (cwm/fastgen/forward.py:543; the reference
    has no scale, which is `scale=None`)."""

    replayable = True

    def __init__(self, vocab_size: int, dim: int, scale: Optional[float] = None, tensor: str = "weight", streams: int = 1) -> None:
        """`tensor`: the table's local name ("" where the folder names it by the part's prefix alone).  `streams`: a
        residual of several streams starts with the scaled row in every one of them, [T, streams * D]."""
        self.vocab_size = vocab_size
        self.dim = dim
        self.scale = 1.0 if scale is None else float(scale)
        self.tensor = tensor
        self.streams = streams

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.tensor: TensorSpec((self.vocab_size, self.dim))}

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.table = tensors[self.tensor].contiguous()

    def forward(self, batch: Any) -> torch.Tensor:
        if self.streams > 1:
            return ops.embedding_streams(batch.tokens, self.table, self.streams, self.scale)
        return ops.embedding(batch.tokens, self.table, self.scale)


class NormedTokenEmbedding(TokenEmbedding):
    """The table's rows, normalised: h = norm(scale * table[tokens]).  `norm` is any norm part that can
    normalise rows where they lie (`normalize_`); its tensors carry `norm_prefix` after the table's name."""

    def __init__(
        self, vocab_size: int, dim: int, norm: PartChoice, scale: Optional[float] = None, tensor: str = "weight", norm_prefix: str = "norm.",
    ) -> None:
        super().__init__(vocab_size, dim, scale, tensor)
        self.norm = norm.build("norm")
        self.norm_prefix = norm_prefix
        if not hasattr(self.norm, "normalize_"):
            raise TypeError(f"the norm {norm.name!r} cannot normalise rows in place")

    @property
    def replayable(self) -> bool:  # type: ignore[override]
        return self.norm.replayable

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = super().tensor_specs()
        for name, spec in self.norm.tensor_specs().items():
            specs[self.norm_prefix + name] = spec
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        n = len(self.norm_prefix)
        self.norm.bind({name[n:]: t for name, t in tensors.items() if name != self.tensor and name.startswith(self.norm_prefix)}, runtime)

    def forward(self, batch: Any) -> torch.Tensor:
        return self.norm.normalize_(super().forward(batch))


class LinearHead(Head):
    """logits = x W^T in float32 (cwm/fastgen/forward.py:820-821).  A model whose head is its embedding table
    gives this part the embedding's prefix: both then name the same tensor."""

    replayable = True

    def __init__(self, vocab_size: int, dim: int, tensor: str = "weight") -> None:
        self.vocab_size = vocab_size
        self.dim = dim
        self.tensor = tensor

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.tensor: TensorSpec((self.vocab_size, self.dim))}

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.weights = LinearWeights(tensors[self.tensor], stream_copy=runtime.stream_copies)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.weights(x, out_dtype=torch.float32)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("embedding", "normed_embedding", NormedTokenEmbedding)
register_part("head", "linear_head", LinearHead)
