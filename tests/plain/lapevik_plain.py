"""Plain implementation of every mechanism of the Lapevik decoder.

Whole sequences, no cache, one function per mechanism, nothing imported from the
product package.  All arithmetic runs in the dtype of the inputs (tests use float64
on the CPU).  With `rounded=True` the values that a bfloat16 run stores in 16 bits
(inputs and results of matrix products, the convolution's output, cached rows,
attention probabilities) are rounded to bfloat16 on the way, while everything that
the design keeps in 32 bits (norms, scores, router, residual sum, recurrent state
and what enters it) stays wide: the distance of such a run from the exact one is
what bfloat16 storage costs for the weights and tokens at hand.

Notation.  D model width, T tokens of one sequence, positions 0..T-1.

  group norm      y = w * x_g / sqrt(mean(x_g^2) + eps) for each of `groups` equal consecutive parts x_g of x
  layer           x += norm1(mixer(shift(x)));  x += norm2(ff(x))  (the second only where the layer has a ff)
  token shift     s_t = x_t + (x_(t-1) - x_t) * mu,  x_(-1) = 0
  state space     u = W_in s = [z | xs | B | C | dt];  (xs, B, C) <- silu(conv(xs, B, C));  dt <- softplus(dt + dt_bias)
                  S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t xs_t^T;  y_t = S_t^T C_t + D xs_t   (per head)
                  out = W_o (w * groupnorm(y * silu(z)))
  latent attn     cq = rms(W_dq s) * w_q;  q = W_uq cq, per head [nope | rope]
                  (c | kr) = W_dkv s;  c <- rms(c) * w_kv;  k_h = [W_uk,h c | rot(kr)],  v_h = W_uv,h c
                  a_h = softmax_(j<=i)(scale * q_h,i . k_h,j) v_h;  out = W_o (a * sigmoid(W_g s))
  experts         z = W_r x (wide); the `top` largest; weights softmax over those; sum_e w_e W_down,e (silu(W_gate,e x) * W_up,e x)
"""

from __future__ import annotations

import math
import re
from typing import Dict, List, Mapping, Optional, Sequence, Tuple

import torch


def _bf16(x: torch.Tensor, on: bool) -> torch.Tensor:
    return x.to(torch.bfloat16).to(x.dtype) if on else x


def linear(x: torch.Tensor, w: torch.Tensor, rounded: bool = False) -> torch.Tensor:
    """W x for every row of x, W stored [out, in]."""
    return _bf16(_bf16(x, rounded) @ w.T, rounded)


def group_rms_norm(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """Each of `groups` equal consecutive parts of the last axis is divided by its own root mean square."""
    shape = x.shape
    parts = x.reshape(*shape[:-1], groups, shape[-1] // groups)
    parts = parts / torch.sqrt((parts * parts).mean(dim=-1, keepdim=True) + eps)
    return parts.reshape(shape) * w


def token_shift(x: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    """s_t = x_t + (x_(t-1) - x_t) * mu with zeros before the first token."""
    prev = torch.cat([torch.zeros_like(x[:1]), x[:-1]], dim=0)
    return x + (prev - x) * mu


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def causal_conv(u: torch.Tensor, w: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Per channel: out_t = b + sum_k w[:, k] * u_(t - (taps - 1 - k)); inputs before the start are zero."""
    n, _ = u.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype), u], dim=0)
    out = b.expand(n, -1).clone()
    for k in range(taps):
        out = out + padded[k : k + n] * w[:, k]
    return out


def state_space(
    s: torch.Tensor, t: Mapping[str, torch.Tensor], heads: int, vdim: int, state: int, groups: int, norm_groups: int,
    eps: float, rounded: bool = False,
) -> torch.Tensor:
    """The selective state-space mixer, token by token."""
    inner = heads * vdim
    gn = groups * state
    u = linear(s, t["in"], rounded)
    z, xbc, dt = u[:, :inner], u[:, inner : 2 * inner + 2 * gn], u[:, 2 * inner + 2 * gn :]
    xbc = _bf16(silu(causal_conv(xbc, t["conv"], t["conv.b"])), rounded)
    xs = xbc[:, :inner].reshape(-1, heads, vdim)
    bmat = xbc[:, inner : inner + gn].reshape(-1, groups, state)
    cmat = xbc[:, inner + gn :].reshape(-1, groups, state)
    dt = softplus(dt + t["dt_bias"])
    decay = torch.exp(-torch.exp(t["A_log"]) * dt)  # [T, heads]
    per_group = heads // groups
    y = torch.zeros_like(xs)
    carry = torch.zeros(heads, state, vdim, dtype=s.dtype)
    for i in range(s.shape[0]):
        for h in range(heads):
            g = h // per_group
            carry[h] = decay[i, h] * carry[h] + dt[i, h] * torch.outer(bmat[i, g], xs[i, h])
            y[i, h] = carry[h].T @ cmat[i, g] + t["D"][h] * xs[i, h]
    y = y.reshape(-1, inner) * silu(z)
    y = group_rms_norm(y, t["norm"], norm_groups, eps)
    return linear(y, t["o"], rounded)


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """Element 2i and 2i+1 of the first `dims` elements of the last axis turn by positions * base^(-2i/dims);
    x is [T, ..., n] and the rest of the last axis passes unchanged."""
    out = x.clone()
    for i in range(dims // 2):
        angle = positions.to(x.dtype) * (base ** (-2.0 * i / dims))
        while angle.dim() < x.dim() - 1:
            angle = angle.unsqueeze(-1)
        cos, sin = torch.cos(angle), torch.sin(angle)
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = a * cos - b * sin
        out[..., 2 * i + 1] = b * cos + a * sin
    return out


def latent_attention(
    s: torch.Tensor, t: Mapping[str, torch.Tensor], heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, scale: float,
    rot_base: float, rot_dims: int, eps: float, rounded: bool = False,
) -> torch.Tensor:
    n = s.shape[0]
    positions = torch.arange(n)
    cq = _bf16(group_rms_norm(linear(s, t["dq"], rounded), t["dq.norm"], 1, eps), rounded)
    q = linear(cq, t["uq"], rounded).reshape(n, heads, dim + rot_dim)
    q_nope, q_rope = q[..., :dim], _bf16(rotate_pairs(q[..., dim:], positions, rot_base, rot_dims), rounded)
    down = linear(s, t["dkv"], rounded)
    c = _bf16(group_rms_norm(down[:, :kv_rank], t["dkv.norm"], 1, eps), rounded)
    k_rope = _bf16(rotate_pairs(down[:, kv_rank:], positions, rot_base, rot_dims), rounded)
    k_nope = linear(c, t["uk"], rounded).reshape(n, heads, dim)
    v = linear(c, t["uv"], rounded).reshape(n, heads, vdim)
    scores = (torch.einsum("ihd,jhd->hij", q_nope, k_nope) + torch.einsum("ihd,jd->hij", q_rope, k_rope)) * scale
    visible = positions[None, :] <= positions[:, None]
    scores = scores.masked_fill(~visible, float("-inf"))
    weights = _bf16(torch.softmax(scores, dim=-1), rounded)
    mixed = _bf16(torch.einsum("hij,jhd->ihd", weights, v), rounded).reshape(n, heads * vdim)
    gate = torch.sigmoid(linear(s, t["g"], rounded))
    return linear(_bf16(mixed * gate, rounded), t["o"], rounded)


def routed_experts(x: torch.Tensor, t: Mapping[str, torch.Tensor], experts: int, top: int, rounded: bool = False) -> torch.Tensor:
    """Each token's `top` experts by router logit, weighted by the softmax over those logits alone."""
    logits = _bf16(x, rounded) @ t["router"].T
    chosen = torch.topk(logits, top, dim=-1)
    weights = torch.softmax(chosen.values, dim=-1)
    out = torch.zeros_like(x)
    for e in range(experts):
        hidden = _bf16(silu(linear(x, t[f"e{e}.gate"], rounded)) * linear(x, t[f"e{e}.up"], rounded), rounded)
        y = linear(hidden, t[f"e{e}.down"], rounded)
        w = (weights * (chosen.indices == e)).sum(dim=-1, keepdim=True)
        out = out + w * y
    return out


def mixer_kind(layer_type: str) -> str:
    """'name_2' is a second set of sizes for mixer 'name'."""
    return re.sub(r"_\d+$", "", layer_type)


def _sub(weights: Mapping[str, torch.Tensor], prefix: str, dtype: torch.dtype) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.to(dtype) for k, v in weights.items() if k.startswith(prefix)}


def forward(
    weights: Mapping[str, torch.Tensor], config: Mapping, tokens: Sequence[int], dtype: torch.dtype = torch.float64, rounded: bool = False,
    layer_outputs: Optional[List[torch.Tensor]] = None,
) -> torch.Tensor:
    """Logits [T, vocab] of one sequence; `layer_outputs` receives the residual stream after every layer."""
    eps, groups = float(config["norm"]["eps"]), int(config["norm"]["groups"])
    embed = weights["embed"].to(dtype)
    x = embed[torch.as_tensor(list(tokens), dtype=torch.long)]
    x = group_rms_norm(x, weights["embed.norm"].to(dtype), groups, eps)
    for i, layer in enumerate(config["layers"]):
        m = layer["mixer"]
        s = token_shift(x, weights[f"l{i}.shift"].to(dtype))
        t = _sub(weights, f"l{i}.mix.", dtype)
        kind = mixer_kind(layer["type"])
        if kind == "mamba2":
            y = state_space(s, t, m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"], eps, rounded)
        elif kind == "latent_attention":
            y = latent_attention(
                s, t, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], float(m["scale"]),
                float(m["rot"]["base"]), int(m["rot"]["dims"]), eps, rounded,
            )
        else:
            raise ValueError(f"unknown mixer {layer['type']!r}")
        x = x + group_rms_norm(y, weights[f"l{i}.norm1"].to(dtype), groups, eps)
        if layer.get("mlp") is not None:
            mlp = layer["mlp"]
            y = routed_experts(x, _sub(weights, f"l{i}.mlp.", dtype), mlp["router"]["experts"], mlp["router"]["top"], rounded)
            x = x + group_rms_norm(y, weights[f"l{i}.norm2"].to(dtype), groups, eps)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    x = _bf16(group_rms_norm(x, weights["final.norm"].to(dtype), groups, eps), rounded)
    return x @ embed.T
