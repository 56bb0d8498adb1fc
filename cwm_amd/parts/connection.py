"""Connections between a sublayer and a residual of one or several streams."""

from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from .. import ops
from .base import Connection, Runtime, TensorSpec, register_part
from .norm import StreamUpdate


class ResidualSum(Connection):
    """x <- x + y on a single stream; the sublayer reads x itself.  No tensors."""

    replayable = True
    streams = 1

    def update(self, y: torch.Tensor) -> StreamUpdate:
        return StreamUpdate(y)


class HyperConnection(Connection):
    """The residual is `streams` vectors x_1 .. x_S a token.  The sublayer reads u = sum_s in[s] x_s; its result y
    changes all streams at once from the old ones, x_t <- sum_s mix[s, t] x_s + out[t] y (`mix` is indexed
    [from, to]).  Tensors `in` [S], `out` [S], `mix` [S, S]; all arithmetic on them is float32."""

    replayable = True

    def __init__(self, streams: int) -> None:
        if not 1 <= streams <= ops.MAX_STREAMS:
            raise ValueError(f"{streams} streams: the kernels take 1..{ops.MAX_STREAMS}")
        self.streams = streams

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        s = self.streams
        return {
            "in": TensorSpec((s,), init="ones", precision="stored"),
            "out": TensorSpec((s,), init="ones", precision="stored"),
            "mix": TensorSpec((s, s), init="identity", precision="stored"),
        }

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self._in = tensors["in"].float().contiguous()
        self._out = tensors["out"].float().contiguous()
        self._mix = tensors["mix"].float().contiguous()

    def in_coef(self) -> Optional[torch.Tensor]:
        return self._in

    def update(self, y: torch.Tensor) -> StreamUpdate:
        return StreamUpdate(y, self._mix, self._out)


register_part("connection", "residual_sum", ResidualSum)
register_part("connection", "hyper_connection", HyperConnection)
