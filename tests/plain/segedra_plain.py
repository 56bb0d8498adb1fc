"""The Segedra decoder, plainly: whole sequences, no cache, no batching, one function per mechanism, written from the
design's equations and sharing nothing with the product.

In this file's notation, for one sequence of n tokens and a residual of S streams X[s] (each [n, D]):

    X[s]      = scale_e * E[token]                         for every stream s
    sublayer:   u  = sum_s a[s] X[s]                        a = hc.in
                y  = f(u / sqrt(mean(u^2) + eps) * (1 + w))
                X'[t] = sum_s M[s, t] X[s] + b[t] y         M = hc.mix (from, to), b = hc.out
    without streams in the configuration: x += f(norm(x)), the same with S = 1 and a = b = M = 1
    attention:  q, k over all heads divided by their root mean square, times a weight per element; the first
                `rot.dims` elements of each head turned in adjacent pairs by position * base^(-2i/dims);
                p_ij = exp(scale q_i.k_j) / (sum_(j' in window) exp(scale q_i.k_j') + exp(sink_h)),  0 <= i - j < mask.size
    dense:      W_down relu(W_up h)^2
    experts:    s = softmax(W_r h); chosen = the `top` largest of s + correction; out = sum_e router.scale * s_e * expert_e(h);
                expert(h) = W_down (g * sigmoid(1.702 g) * (u + 1)), g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit)
    loop:       layers start .. stop - 1 run `times` times in a row
    logits    = E (norm_final(sum_s X[s]))

`rounded=True` rounds to bfloat16 wherever an engine that computes in bfloat16 stores a tensor of that type (the inputs
and results of matrix products, rotated queries and keys, cached values, attention weights and outputs), still in
float64 arithmetic: what bfloat16 storage alone costs.
"""

from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional

import torch

EXPERT_SLOPE = 1.702


def _bf16(x: torch.Tensor, on: bool) -> torch.Tensor:
    return x.to(torch.bfloat16).to(x.dtype) if on else x


def linear(x: torch.Tensor, w: torch.Tensor, rounded: bool = False) -> torch.Tensor:
    """W x for every row of x, W stored [out, in]."""
    return _bf16(_bf16(x, rounded) @ w.T, rounded)


def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float, one_plus: bool) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    if w is None:
        return y
    return y * (1 + w) if one_plus else y * w


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, base: float, dims: int) -> torch.Tensor:
    """x [n, heads, d]: elements (2i, 2i + 1), i < dims / 2, of every head turned by position * base^(-2i / dims)."""
    out = x.clone()
    for i in range(dims // 2):
        angle = positions.to(x.dtype) * base ** (-2.0 * i / dims)
        c, s = torch.cos(angle)[:, None], torch.sin(angle)[:, None]
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def sink_softmax(scores: torch.Tensor, sink: Optional[torch.Tensor]) -> torch.Tensor:
    """Rows of scores (-inf where masked) -> weights whose denominator also holds exp(sink)."""
    top = scores.max(-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink.reshape(1, 1).expand_as(top))
    e = torch.exp(scores - top)
    denom = e.sum(-1, keepdim=True)
    if sink is not None:
        denom = denom + torch.exp(sink - top)
    return e / denom


def attention(h: torch.Tensor, t: Mapping[str, torch.Tensor], m: Mapping, eps: float, rounded: bool = False) -> torch.Tensor:
    n = h.shape[0]
    heads, kv, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = linear(h, t["q"], rounded), linear(h, t["k"], rounded), linear(h, t["v"], rounded)
    q = rms_norm(q, t.get("q.norm"), eps, one_plus=False).reshape(n, heads, d)
    k = rms_norm(k, t.get("k.norm"), eps, one_plus=False).reshape(n, kv, d)
    v = v.reshape(n, kv, dv)
    positions = torch.arange(n)
    rot = m.get("rot")
    if rot is not None and rot["dims"] > 0:
        q = rotate_pairs(q, positions, rot["base"], rot["dims"])
        k = rotate_pairs(k, positions, rot["base"], rot["dims"])
    q, k = _bf16(q, rounded), _bf16(k, rounded)
    distance = positions[:, None] - positions[None, :]
    seen = distance >= 0
    if m.get("mask") is not None:
        seen = seen & (distance < m["mask"]["size"])
    out = torch.zeros(n, heads, dv, dtype=h.dtype)
    for head in range(heads):
        g = head // (heads // kv)
        scores = (q[:, head] @ k[:, g].T) * m["scale"]
        scores = scores.masked_fill(~seen, -math.inf)
        weights = sink_softmax(scores, t["sink"][head] if "sink" in t else None)
        out[:, head] = _bf16(weights, rounded) @ v[:, g]
    return linear(_bf16(out.reshape(n, heads * dv), rounded), t["o"], rounded)


def dense_feed_forward(h: torch.Tensor, t: Mapping[str, torch.Tensor], rounded: bool = False) -> torch.Tensor:
    return linear(torch.relu(linear(h, t["up"], rounded)) ** 2, t["down"], rounded)


def route(h: torch.Tensor, t: Mapping[str, torch.Tensor], top: int, scale: float, rounded: bool = False, margins: Optional[list] = None):
    """(chosen [n, top], weights [n, top]): scores over all experts; the correction counts for the choice only.
    `margins` receives, per token, how clear the choice was: by how much the last chosen expert's choice score leads
    the first one left out, over how far a relative change of the logits by 1 could move the two scores
    (d s_e = s_e (d z_e - sum_j s_j d z_j), so at most about (s_a + s_b) * |z|)."""
    logits = _bf16(h, rounded) @ t["router"].T
    scores = torch.softmax(logits, -1)
    choice = scores + t["correction"] if "correction" in t else scores
    order = torch.sort(choice, dim=-1, descending=True, stable=True)
    chosen = order.indices[:, :top]
    if margins is not None and top < choice.shape[-1]:
        pair = torch.gather(scores, 1, order.indices[:, top - 1 : top + 1]).sum(-1)
        reach = pair * torch.sqrt((logits * logits).mean(-1)) + 1e-30
        margins.append((order.values[:, top - 1] - order.values[:, top]) / reach)
    return chosen, torch.gather(scores, 1, chosen) * scale


def expert(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, limit: float, rounded: bool = False) -> torch.Tensor:
    g = torch.clamp(_bf16(h, rounded) @ gate.T, max=limit)
    u = torch.clamp(_bf16(h, rounded) @ up.T, min=-limit, max=limit)
    return _bf16(g * torch.sigmoid(EXPERT_SLOPE * g) * (u + 1), rounded) @ down.T


def routed_experts(h: torch.Tensor, t: Mapping[str, torch.Tensor], mlp: Mapping, rounded: bool = False, margins: Optional[list] = None) -> torch.Tensor:
    chosen, weights = route(h, t, mlp["router"]["top"], mlp["router"].get("scale", 1.0), rounded, margins)
    out = torch.zeros_like(h)
    for e in range(mlp["router"]["experts"]):
        rows, places = torch.nonzero(chosen == e, as_tuple=True)
        if rows.numel():
            y = expert(h[rows], t[f"e{e}.gate"], t[f"e{e}.up"], t[f"e{e}.down"], mlp["expert"]["limit"], rounded)
            out[rows] += weights[rows, places][:, None] * y
    return out


def read_streams(streams: torch.Tensor, a: Optional[torch.Tensor]) -> torch.Tensor:
    """streams [S, n, D] -> what a sublayer reads."""
    return streams.sum(0) if a is None else torch.einsum("s,snd->nd", a, streams)


def write_streams(streams: torch.Tensor, y: torch.Tensor, mix: Optional[torch.Tensor], b: Optional[torch.Tensor]) -> torch.Tensor:
    """All streams at once from the old ones."""
    if mix is None:
        return streams + y[None]
    return torch.einsum("st,snd->tnd", mix, streams) + b[:, None, None] * y[None]


def layer_order(config: Mapping) -> List[int]:
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    return list(range(loop["start"])) + list(range(loop["start"], loop["stop"])) * loop["times"] + list(range(loop["stop"], n))


def _sub(weights: Mapping[str, torch.Tensor], prefix: str, dtype: torch.dtype) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.to(dtype) for k, v in weights.items() if k.startswith(prefix)}


def forward(
    weights: Mapping[str, torch.Tensor], config: Mapping, tokens: List[int], dtype: torch.dtype = torch.float64, rounded: bool = False,
    after_layers: Optional[list] = None, margins: Optional[list] = None,
) -> torch.Tensor:
    """Logits [n, vocab] of one sequence.  `after_layers` receives the sum of the streams after every layer run,
    `margins` every router's margins of choice (see `route`), one tensor [n] a run of a layer with experts."""
    eps = config["norm"]["eps"]
    table = weights["embed"].to(dtype)
    x = table[torch.tensor(tokens)] * config.get("embedding", {}).get("scale", 1.0)
    hyper = config.get("streams") is not None
    streams = x[None].repeat(config["streams"] if hyper else 1, 1, 1)
    for index in layer_order(config):
        layer, p = config["layers"][index], f"l{index}."
        sublayers = [(1, lambda u: attention(u, _sub(weights, p + "mix.", dtype), layer["mixer"], eps, rounded))]
        if layer.get("mlp") is not None:
            t = _sub(weights, p + "mlp.", dtype)
            if layer["mlp"]["kind"] == "dense":
                sublayers.append((2, lambda u: dense_feed_forward(u, t, rounded)))
            else:
                sublayers.append((2, lambda u: routed_experts(u, t, layer["mlp"], rounded, margins)))
        for number, f in sublayers:
            hc = _sub(weights, p + f"hc{number}.", dtype) if hyper else {}
            u = read_streams(streams, hc.get("in"))
            y = f(_bf16(rms_norm(u, weights[p + f"norm{number}"].to(dtype), eps, one_plus=True), rounded))
            streams = write_streams(streams, y, hc.get("mix"), hc.get("out"))
        if after_layers is not None:
            after_layers.append(streams.sum(0))
    x = _bf16(rms_norm(streams.sum(0), weights["final.norm"].to(dtype), eps, one_plus=True), rounded)
    return x @ table.T
