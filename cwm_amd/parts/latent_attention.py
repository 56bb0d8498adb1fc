"""Causal attention whose keys and values are rebuilt from one cached latent row per token."""

from __future__ import annotations

from typing import Any, Dict, Mapping, Optional

import torch

from .. import ops
from .attention import MAX_HEAD_DIM
from .base import Mixer, PagedKVSpec, PartChoice, PositionEncoding, Runtime, TensorSpec, register_part
from .linear import LinearWeights


class LatentAttention(Mixer):
    """Queries through a latent: cq = rms(W_dq s) w_q, q_h = (W_uq cq)_h = [n_h | r_h] with `head_dim` unrotated and
    `rot_dim` rotated elements.  Keys and values through another: W_dkv s = [c | kr], c <- rms(c) w_kv; head h has
    the key [W_uk,h c | rot(kr)] and the value W_uv,h c; scores scale * q.k over the causal past, softmax, and
    the heads' results times sigmoid(W_g s) go through W_o.

    Only [rot(kr) | c] is cached, one row a token, and attention runs on those rows directly: since
    n_h . (W_uk,h c) = (W_uk,h^T n_h) . c, head h asks with [rot(r_h) | W_uk,h^T n_h], all heads read the one
    row as key and as value, and W_uv,h is applied to the weighted sum of latents afterwards.  That is
    attention with one key/value head of size rot_dim + kv_rank, which the paged attention kernels serve; the
    rotated part leads the row so that the rotation's pairs start at an even element.  The position encoding
    turns the first elements of the rotated part (its table may be shorter than rot_dim / 2: the rest of the
    part and the latent have frequency 0 and pass unchanged)."""

    def __init__(
        self, dim: int, n_heads: int, head_dim: int, rot_dim: int, v_dim: int, kv_rank: int, q_rank: int, scale: float, eps: float,
        position_encoding: Optional[PartChoice] = None,
    ) -> None:
        self.row = rot_dim + kv_rank  # a cached row, and the size of the one key/value head
        if self.row > MAX_HEAD_DIM:
            raise ValueError(f"a cached row of {rot_dim} + {kv_rank} elements is more than the {MAX_HEAD_DIM} the attention kernels take")
        if rot_dim % 2 != 0 or self.row % 2 != 0:
            raise ValueError("the rotated part and the cached row need even sizes")
        self.dim, self.n_heads, self.head_dim, self.rot_dim, self.v_dim = dim, n_heads, head_dim, rot_dim, v_dim
        self.kv_rank, self.q_rank, self.scale = kv_rank, q_rank, float(scale)
        norm = lambda n, name: PartChoice("group_rmsnorm", {"dim": n, "eps": eps, "groups": 1, "tensor": name}).build("norm")  # noqa: E731
        self.q_norm = norm(q_rank, "dq.norm")
        self.kv_norm = norm(kv_rank, "dkv.norm")
        self.position_encoding: Optional[PositionEncoding] = (
            position_encoding.build("position_encoding") if position_encoding is not None else None
        )

    @property
    def replayable(self) -> bool:  # type: ignore[override]
        return self.position_encoding is None or self.position_encoding.replayable

    def cache_spec(self) -> PagedKVSpec:
        return PagedKVSpec(n_kv_heads=1, head_dim=self.row, window=None)

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        h = self.n_heads
        return {
            "dq": TensorSpec((self.q_rank, self.dim)),
            **self.q_norm.tensor_specs(),
            "uq": TensorSpec((h * (self.head_dim + self.rot_dim), self.q_rank)),
            "dkv": TensorSpec((self.kv_rank + self.rot_dim, self.dim)),
            **self.kv_norm.tensor_specs(),
            "uk": TensorSpec((h * self.head_dim, self.kv_rank)),
            "uv": TensorSpec((h * self.v_dim, self.kv_rank)),
            "g": TensorSpec((h * self.v_dim, self.dim)),
            "o": TensorSpec((self.dim, h * self.v_dim)),
        }

    def bind(self, tensors: Mapping[str, torch.Tensor], runtime: Runtime) -> None:
        super().bind(tensors, runtime)
        self.q_norm.bind({"dq.norm": tensors["dq.norm"]}, runtime)
        self.kv_norm.bind({"dkv.norm": tensors["dkv.norm"]}, runtime)
        h, hd, rd, kr = self.n_heads, self.head_dim, self.rot_dim, self.kv_rank
        dkv = tensors["dkv"]
        # one product for everything that reads s: [kr | c] (the rotated part first, as the cache keeps it), cq, gate
        self.down = LinearWeights.joined(
            [torch.cat([dkv[kr:], dkv[:kr]], dim=0), tensors["dq"], tensors["g"]], [None, None, None], stream_copy=runtime.stream_copies,
        )
        # the rows of W_uq head by head as [r_h | n_h], so that the rotated part leads here too
        uq = tensors["uq"].reshape(h, hd + rd, self.q_rank)
        self.up_q = LinearWeights(torch.cat([uq[:, hd:], uq[:, :hd]], dim=1).reshape(h * (hd + rd), self.q_rank), stream_copy=runtime.stream_copies)
        self.w_uk = tensors["uk"].reshape(h, hd, kr).transpose(1, 2).contiguous()  # [h, kv_rank, head_dim]: n_h -> W_uk,h^T n_h
        self.w_uv = tensors["uv"].reshape(h, self.v_dim, kr).contiguous()  # [h, v_dim, kv_rank]: sum of latents -> value
        self.w_o = LinearWeights(tensors["o"], stream_copy=runtime.stream_copies)
        table = None
        if self.position_encoding is not None:
            self.position_encoding.bind({}, runtime)
            if self.position_encoding.rotary_pairing() != "adjacent":
                raise ValueError("the latent attention rotates adjacent pairs")
            table = self.position_encoding.rotary_table()
        self.table = None
        if table is not None:
            if 2 * table.numel() > rd:
                raise ValueError(f"a rotation of {2 * table.numel()} elements does not fit the rotated part of {rd}")
            self.table = torch.zeros(self.row // 2, dtype=torch.float32, device=runtime.device)
            self.table[: table.numel()] = table

    def forward(self, x: torch.Tensor, batch: Any, cache: Any, write_cache: bool = True) -> torch.Tensor:
        h, hd, rd, kr, row = self.n_heads, self.head_dim, self.rot_dim, self.kv_rank, self.row
        n = x.shape[0]
        down = self.down(x)  # [T, row + q_rank + h * v_dim]
        key_rows = down[:, :row]
        self.kv_norm.normalize_(key_rows[:, rd:])
        cq = self.q_norm.forward(down[:, row : row + self.q_rank], None)
        q = self.up_q(cq).unflatten(1, (h, hd + rd))
        # what each head asks the cached rows with: [r_h | W_uk,h^T n_h]
        ask = ops.absorb_queries(q, rd, self.w_uk)  # [T, h, row]
        keys = key_rows.unflatten(1, (1, row))
        if write_cache:
            ops.rope_kv_write(ask, keys, None, batch.positions, self.table)  # rotation in place
            ops.rope_kv_write(keys, keys, keys, batch.positions, None, cache.cache, cache.block_table, batch.seq_of_token)  # the row as key and value
        else:
            ops.rope_kv_write(ask, None, None, batch.positions, self.table)
        mixed = ops.paged_attention(ask, cache.cache, cache.block_table, batch, None, self.scale).unflatten(1, (h, row))
        values = ops.expand_values(mixed, rd, self.w_uv)  # [T, h * v_dim]
        gated = ops.sigmoid_mul(values, down[:, row + self.q_rank :])
        return self.w_o(gated, partials_ok=True)


register_part("mixer", "latent_attention", LatentAttention)
