"""Entry points of the routing kernels and the grouped product (`csrc/routed.hip`): routed experts, and products
in which every head has a weight matrix of its own."""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import build as _build

MAX_ROUTE_TOP = 16  # csrc/routed.hip: ROUTE_MAX_TOP
MAX_EXPERTS = 256  # csrc/routed.hip: ROUTE_MAX_EXPERTS
TILE_ROWS = 16  # rows of a tile of the grouped product
MEDIUM_ROWS = 64  # from so many rows an expert (on average) a block of the grouped product takes 4 row tiles,
WIDE_ROWS = 256  # and from so many, 8


def _base():
    from . import KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream

    return KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream


def route_top(
    logits: torch.Tensor, top: int, scores: str = "softmax_chosen", correction: Optional[torch.Tensor] = None, scale: float = 1.0,
    renormalize: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """float32 router logits [T, E] -> (chosen int32 [T, top], weights float32 [T, top]), the chosen in falling order
    of what they were chosen by (the lower index first among equals).
    `scores` "softmax_chosen": the `top` largest logits, weighted by the softmax over those alone.
    `scores` "softmax_all": s = softmax over all experts; the `top` largest of s + `correction` (float32 [E], None for
    none) are chosen; their weights are `scale` * s (the correction is no part of a weight), divided by the sum of
    the chosen s first if `renormalize`."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(logits, correction)
    if scores not in ("softmax_chosen", "softmax_all"):
        raise KernelError(f"router scores {scores!r}: 'softmax_chosen' and 'softmax_all' are known")
    if scores == "softmax_chosen" and (correction is not None or scale != 1.0 or renormalize):
        raise KernelError("a correction, a scale and renormalised weights belong to router scores over all experts")
    if correction is not None and (correction.dtype != torch.float32 or correction.shape != (logits.shape[-1],) or not correction.is_contiguous()):
        raise KernelError("the router's correction must be a contiguous float32 tensor, one value an expert")
    if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous():
        raise KernelError("router logits must be a contiguous float32 [T, E] tensor")
    n, e = logits.shape
    if not 1 <= top <= min(e, MAX_ROUTE_TOP):
        raise KernelError(f"{top} of {e} experts: the kernel takes 1..{min(e, MAX_ROUTE_TOP)}")
    chosen = torch.empty((n, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((n, top), dtype=torch.float32, device=logits.device)
    lib = _build.load("routed")
    _check(
        lib,
        lib.cwm_route_top(
            _ptr(logits), _ptr(chosen), _ptr(weights), ctypes.c_int(n), ctypes.c_int(e), ctypes.c_int(top),
            ctypes.c_int(int(scores == "softmax_all")), _ptr(correction), ctypes.c_float(scale), ctypes.c_int(int(renormalize)), _stream(),
        ),
    )
    return chosen, weights


@dataclass
class ExpertGroups:
    """The step's (token, choice) pairs grouped by expert in tiles of 16 rows."""

    row_token: torch.Tensor  # int32 [tiles * 16]: the token of each row, -1 in the padding
    pair_row: torch.Tensor  # int32 [T * top]: the row of each pair
    tile_expert: torch.Tensor  # int32 [tiles]: the expert of each tile, -1 for tiles not in use
    n_tiles: int
    tiles_a_block: int  # row tiles that one block of the grouped product takes (an expert's tiles start at a multiple)
    top: int


def _tiles_a_block(rows: float) -> int:
    return 8 if rows >= WIDE_ROWS else 4 if rows >= MEDIUM_ROWS else 1


def group_by_expert(chosen: torch.Tensor, n_experts: int) -> ExpertGroups:
    """Group the pairs of `chosen` (int32 [T, top]) by expert.  The lists have a size that depends on T, top and
    the number of experts alone, so no count has to come to the host."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(chosen)
    _i32(chosen, "chosen")
    if chosen.dim() != 2:
        raise KernelError("chosen must be [T, top]")
    if not 1 <= n_experts <= MAX_EXPERTS:
        raise KernelError(f"{n_experts} experts: the kernel takes up to {MAX_EXPERTS}")
    n, top = chosen.shape
    pairs = n * top
    align = _tiles_a_block(pairs / n_experts)
    n_tiles = -(-pairs // TILE_ROWS) + n_experts * align
    lists = torch.empty(n_tiles * TILE_ROWS + pairs + n_tiles, dtype=torch.int32, device=chosen.device)
    a, b = n_tiles * TILE_ROWS, n_tiles * TILE_ROWS + pairs
    groups = ExpertGroups(lists[:a], lists[a:b], lists[b:], n_tiles, align, top)
    lib = _build.load("routed")
    _check(
        lib,
        lib.cwm_group_by_expert(
            _ptr(chosen), ctypes.c_int(n), ctypes.c_int(top), ctypes.c_int(n_experts), _ptr(groups.row_token), _ptr(groups.pair_row),
            _ptr(groups.tile_expert), ctypes.c_int(n_tiles), ctypes.c_int(align), _stream(),
        ),
    )
    return groups


def _grouped(
    a: torch.Tensor, a_ld: int, a_batch: int, groups: Optional[ExpertGroups], w0: torch.Tensor, w1: Optional[torch.Tensor],
    out: torch.Tensor, out_ld: int, out_batch: int, n_rows: int, n_batch: int, tiles_a_block: int,
    activation: Optional["GatedActivation"] = None,
) -> None:
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(a, w0, w1, out)
    if w0.dim() != 3 or not w0.is_contiguous() or w0.dtype != a.dtype or (w1 is not None and (w1.shape != w0.shape or not w1.is_contiguous() or w1.dtype != a.dtype)):
        raise KernelError("grouped weights must be contiguous [experts, N, K] tensors of the rows' type")
    _, n, k = w0.shape
    lib = _build.load("routed")
    _check(
        lib,
        lib.cwm_grouped_product(
            _ptr(a), ctypes.c_long(a_ld), ctypes.c_long(a_batch), ctypes.c_int(_code(a.dtype)),
            _ptr(groups.row_token if groups is not None else None), _ptr(w0), _ptr(w1), ctypes.c_long(n * k),
            _ptr(groups.tile_expert if groups is not None else None), ctypes.c_int(groups.n_tiles if groups is not None else 0),
            ctypes.c_int(n_batch), _ptr(out), ctypes.c_int(_code(out.dtype)), ctypes.c_long(out_ld), ctypes.c_long(out_batch),
            ctypes.c_int(n_rows), ctypes.c_int(n), ctypes.c_int(k), ctypes.c_int(tiles_a_block),
            ctypes.c_int(activation.code() if activation is not None else 0), ctypes.c_float(activation.alpha if activation is not None else 1.0),
            ctypes.c_float(activation.limit if activation is not None else 0.0), _stream(),
        ),
    )


@dataclass(frozen=True)
class GatedActivation:
    """What a gated feed-forward makes of g = W_gate x and u = W_up x.
    "silu": silu(g) * u.
    "clamped_swish": g' * sigmoid(alpha * g') * (u' + 1) with g' = min(g, limit) and u' = clamp(u, -limit, limit)."""

    kind: str = "silu"
    alpha: float = 1.0
    limit: float = 0.0

    def code(self) -> int:
        kinds = {"silu": 0, "clamped_swish": 1}
        if self.kind not in kinds:
            raise ValueError(f"gated activation {self.kind!r}: known are {', '.join(kinds)}")
        return kinds[self.kind]


def grouped_gate_up(
    x: torch.Tensor, groups: ExpertGroups, gate: torch.Tensor, up: torch.Tensor, activation: Optional[GatedActivation] = None
) -> torch.Tensor:
    """act(W_gate,e x_t, W_up,e x_t) for every pair's row, act = silu(g) * u unless `activation` says otherwise:
    `x` [T, D] contiguous, weights [E, F, D]; returns [rows, F] in the type of `x` (rows of the padding are not
    written)."""
    KernelError = _base()[0]
    if x.dim() != 2 or not x.is_contiguous() or gate.shape[2] != x.shape[1]:
        raise KernelError("x must be a contiguous [T, D] tensor that fits the experts' weights")
    out = torch.empty((groups.n_tiles * TILE_ROWS, gate.shape[1]), dtype=x.dtype, device=x.device)
    _grouped(x, x.shape[1], 0, groups, gate, up, out, gate.shape[1], 0, groups.n_tiles * TILE_ROWS, 1, groups.tiles_a_block, activation)
    return out


def grouped_linear(rows: torch.Tensor, groups: ExpertGroups, weight: torch.Tensor) -> torch.Tensor:
    """W_e row for every row of the list (`rows` [rows, F] as `grouped_gate_up` leaves them, `weight` [E, D, F]):
    float32 [rows, D]."""
    KernelError = _base()[0]
    if rows.dim() != 2 or not rows.is_contiguous() or weight.shape[2] != rows.shape[1] or rows.shape[0] != groups.n_tiles * TILE_ROWS:
        raise KernelError("the rows do not fit the list or the experts' weights")
    out = torch.empty((rows.shape[0], weight.shape[1]), dtype=torch.float32, device=rows.device)
    identity = ExpertGroups(_identity_rows(rows.shape[0], rows.device), groups.pair_row, groups.tile_expert, groups.n_tiles, groups.tiles_a_block, groups.top)
    _grouped(rows, rows.shape[1], 0, identity, weight, None, out, weight.shape[1], 0, rows.shape[0], 1, groups.tiles_a_block)
    return out


_identity: dict = {}


def _identity_rows(n: int, device: torch.device) -> torch.Tensor:
    """0..n-1 as int32 on the device (kept: the same list serves every step of that many rows)."""
    key = (device, n)
    t = _identity.get(key)
    if t is None:
        if len(_identity) > 64:
            _identity.clear()
        t = _identity[key] = torch.arange(n, dtype=torch.int32, device=device)
    return t


def combine_routed(rows: torch.Tensor, groups: ExpertGroups, weights: torch.Tensor) -> torch.Tensor:
    """out[t] = sum_k weights[t, k] * rows[row of pair (t, k)], added in the order of k: float32 [T, D]."""
    KernelError, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
    _need_gpu(rows, weights)
    if rows.dtype != torch.float32 or rows.dim() != 2 or not rows.is_contiguous():
        raise KernelError("the experts' rows must be a contiguous float32 tensor")
    if weights.dtype != torch.float32 or weights.dim() != 2 or not weights.is_contiguous() or weights.shape[1] != groups.top:
        raise KernelError("weights must be float32 [T, top]")
    n, top = weights.shape
    out = torch.empty((n, rows.shape[1]), dtype=torch.float32, device=rows.device)
    lib = _build.load("routed")
    _check(
        lib,
        lib.cwm_combine_routed(_ptr(rows), ctypes.c_long(rows.shape[1]), _ptr(groups.pair_row), _ptr(weights), _ptr(out), ctypes.c_int(n), ctypes.c_int(top), ctypes.c_int(rows.shape[1]), _stream()),
    )
    return out


def absorb_queries(q: torch.Tensor, lead: int, weight: torch.Tensor) -> torch.Tensor:
    """Per head h: out[t, h] = [q[t, h, :lead] | W_h^T-applied rest], i.e. out[t, h, lead + j] = sum_d weight[h, j, d] * q[t, h, lead + d].
    `q` [T, H, lead + d] contiguous, `weight` [H, n, d]; returns [T, H, lead + n] in the type of `q`."""
    KernelError = _base()[0]
    if q.dim() != 3 or not q.is_contiguous() or weight.dim() != 3 or weight.shape[0] != q.shape[1] or weight.shape[2] != q.shape[2] - lead:
        raise KernelError(f"q {tuple(q.shape)} does not fit the heads' weights {tuple(weight.shape)} after {lead} leading elements")
    n_tokens, heads, width = q.shape
    n = weight.shape[1]
    out = torch.empty((n_tokens, heads, lead + n), dtype=q.dtype, device=q.device)
    if lead and n_tokens:
        # the leading elements of every head as they are: rows of `width` into rows of `lead + n`, one a (token, head)
        _, _check, _code, _i32, _need_gpu, _ptr, _stream = _base()
        lib = _build.load("groupnorm")
        _check(
            lib,
            lib.cwm_copy_columns(
                _ptr(q), ctypes.c_long(width), _ptr(out), ctypes.c_long(lead + n), ctypes.c_int(_code(q.dtype)),
                ctypes.c_long(n_tokens * heads), ctypes.c_int(lead), _stream(),
            ),
        )
    if n_tokens:
        tiles = _tiles_a_block(n_tokens)
        _grouped(q.view(-1)[lead:], heads * width, width, None, weight, None, out.view(-1)[lead:], heads * (lead + n), lead + n, n_tokens, heads, tiles)
    return out


def expand_values(mixed: torch.Tensor, lead: int, weight: torch.Tensor) -> torch.Tensor:
    """Per head h: out[t, h, :] = weight[h] applied to mixed[t, h, lead:], i.e. out[t, h, v] = sum_j weight[h, v, j] * mixed[t, h, lead + j].
    `mixed` [T, H, lead + n] contiguous, `weight` [H, v, n]; returns [T, H * v]."""
    KernelError = _base()[0]
    if mixed.dim() != 3 or not mixed.is_contiguous() or weight.dim() != 3 or weight.shape[0] != mixed.shape[1] or weight.shape[2] != mixed.shape[2] - lead:
        raise KernelError(f"rows {tuple(mixed.shape)} do not fit the heads' weights {tuple(weight.shape)} after {lead} leading elements")
    n_tokens, heads, width = mixed.shape
    v = weight.shape[1]
    out = torch.empty((n_tokens, heads * v), dtype=mixed.dtype, device=mixed.device)
    if n_tokens:
        tiles = _tiles_a_block(n_tokens)
        _grouped(mixed.view(-1)[lead:], heads * width, width, None, weight, None, out, heads * v, v, n_tokens, heads, tiles)
    return out
