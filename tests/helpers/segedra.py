"""Small configurations of the Segedra architecture with weights drawn so that every mechanism matters, the writer of
their model folders, and the plain implementation's logits for them.

Sizes differ wherever two could be equal (query and key/value heads, query/key and value head sizes, the rotated part
of a head, windows, streams, experts and how many a token uses), layers come with a dense feed-forward, with experts
and with none, and the loop covers the start, the middle or nothing."""

from __future__ import annotations

import copy
import json
import os
from typing import Dict, List, Optional

import numpy as np
import torch

from helpers import lapevik  # the same limits: float32 sums in another order; what bfloat16 storage costs
from plain import segedra_plain


def attn(heads, kv_heads, dim, vdim, scale, window=None, rot=None, mlp=None) -> dict:
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        mixer["mask"] = {"size": window}
    if rot is not None:
        mixer["rot"] = {"base": rot[0], "dims": rot[1]}
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def dense(ff: int) -> dict:
    return {"kind": "dense", "ff": ff}


def moe(ff: int, experts: int, top: int, limit: float, scale: float) -> dict:
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top, "scale": scale}}


# three streams; the loop repeats the two middle layers; heads of 12 and 20 share a cached head of 32; a window of one
# key (the query's own) and a layer without a feed-forward; all of an expert layer's experts chosen
TINY_S = {
    "architecture": "Segedra", "vocab": 157, "width": 48, "norm": {"eps": 1e-5}, "embedding": {"scale": 3.0}, "streams": 3,
    "loop": {"start": 1, "stop": 3, "times": 2},
    "layers": [
        attn(6, 2, 12, 20, 0.3, window=7, rot=(1000.0, 8), mlp=dense(56)),
        attn(2, 2, 32, 16, 0.2, window=33, rot=(50000.0, 32), mlp=moe(24, 5, 2, 0.7, 1.5)),
        attn(3, 1, 16, 16, 0.25, window=1, rot=(100.0, 4), mlp=None),
        attn(4, 4, 8, 24, 0.4, window=18, rot=(10000.0, 8), mlp=moe(16, 4, 4, 1.25, 0.8)),
    ],
}
# no streams (a single residual, no connection tensors), no loop; a layer that reads every key, a layer that is not
# rotated; a sharp softmax (large scale), so that single keys, also far ones and those at a window's edge, decide a token
TINY_T = {
    "architecture": "Segedra", "vocab": 101, "width": 40, "norm": {"eps": 1e-6},
    "layers": [
        attn(2, 1, 16, 8, 2.0, window=None, rot=(300.0, 16), mlp=moe(20, 7, 1, 2.0, 2.5)),
        attn(5, 5, 8, 8, 3.0, window=11, rot=None, mlp=dense(30)),
        attn(4, 2, 24, 40, 1.5, window=64, rot=(2000.0, 6), mlp=moe(12, 3, 2, 0.5, 1.0)),
    ],
}
# one stream with connection tensors; the loop runs the first layer three times; heads of 80; a window of two pages
TINY_U = {
    "architecture": "Segedra", "vocab": 211, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 8.0}, "streams": 1,
    "loop": {"start": 0, "stop": 1, "times": 3},
    "layers": [
        attn(2, 1, 80, 48, 0.11, window=16, rot=(250000.0, 40), mlp=moe(32, 6, 3, 1.0, 2.0)),
        attn(8, 2, 16, 32, 0.25, window=50, rot=(10000.0, 16), mlp=dense(96)),
    ],
}
# wider, so that prompts of some hundred tokens take the kernels' shapes for many rows
MEDIUM = {
    "architecture": "Segedra", "vocab": 320, "width": 256, "norm": {"eps": 1e-6}, "embedding": {"scale": 16.0}, "streams": 2,
    "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [
        attn(8, 2, 64, 32, 0.125, window=100, rot=(10000.0, 32), mlp=dense(512)),
        attn(4, 4, 32, 64, 0.18, window=257, rot=(500000.0, 32), mlp=moe(128, 8, 2, 1.0, 2.5)),
    ],
}

ALL = {"tiny_s": TINY_S, "tiny_t": TINY_T, "tiny_u": TINY_U}


def get(name: str) -> dict:
    return copy.deepcopy(ALL[name])


def draw_weights(config: dict, seed: int) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors by name.  Matrices N(0, 1 / fan-in); norm weights around zero (they are applied as 1 + w) and the
    query and key norms around one; sinks of the size of a good score, so that they take a real share of the softmax;
    connection coefficients that mix the streams unevenly; a router whose scores are spread out and a correction
    large enough to change who is chosen."""
    gen = torch.Generator().manual_seed(seed)
    normal = lambda *shape, std=1.0: torch.randn(*shape, generator=gen) * std  # noqa: E731
    uniform = lambda lo, hi, *shape: torch.rand(*shape, generator=gen) * (hi - lo) + lo  # noqa: E731
    matrix = lambda out, inp: normal(out, inp, std=inp ** -0.5)  # noqa: E731
    width, vocab = config["width"], config["vocab"]
    streams = config.get("streams")
    w = {"embed": normal(vocab, width, std=0.5), "final.norm": normal(width, std=0.3)}
    for i, layer in enumerate(config["layers"]):
        m, p = layer["mixer"], f"l{i}."
        numbers = [1] + ([2] if layer["mlp"] is not None else [])
        for q in numbers:
            w[p + f"norm{q}"] = normal(width, std=0.3)
            if streams is not None:
                w[p + f"hc{q}.in"] = uniform(0.3, 1.0, streams)
                w[p + f"hc{q}.out"] = uniform(0.5, 1.5, streams)
                w[p + f"hc{q}.mix"] = torch.eye(streams) * 0.9 + normal(streams, streams, std=0.15)
        q_out, k_out = m["heads"] * m["dim"], m["kv_heads"] * m["dim"]
        w[p + "mix.q"] = matrix(q_out, width)
        w[p + "mix.k"] = matrix(k_out, width)
        w[p + "mix.v"] = matrix(m["kv_heads"] * m["vdim"], width)
        w[p + "mix.q.norm"] = uniform(0.5, 1.5, q_out)
        w[p + "mix.k.norm"] = uniform(0.5, 1.5, k_out)
        w[p + "mix.sink"] = uniform(-1.0, 3.0, m["heads"])
        w[p + "mix.o"] = matrix(width, m["heads"] * m["vdim"])
        mlp = layer["mlp"]
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            w[p + "mlp.up"] = matrix(mlp["ff"], width)
            w[p + "mlp.down"] = matrix(width, mlp["ff"])
        else:
            experts, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
            w[p + "mlp.router"] = normal(experts, width, std=0.5)
            w[p + "mlp.correction"] = uniform(-0.3, 0.3, experts)
            for e in range(experts):
                w[p + f"mlp.e{e}.gate"] = matrix(ff, width) * 1.5  # sums that reach the limit
                w[p + f"mlp.e{e}.up"] = matrix(ff, width) * 1.5
                w[p + f"mlp.e{e}.down"] = matrix(width, ff)
    return {k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}


def make_folder(root, name: str, seed: int = 1, config: Optional[dict] = None, weights: Optional[Dict[str, torch.Tensor]] = None) -> str:
    from safetensors.torch import save_file

    config = config or get(name)
    folder = os.path.join(str(root), f"{name}_{seed}")
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(config, fh)
    save_file(weights if weights is not None else draw_weights(config, seed), os.path.join(folder, "model.safetensors"))
    return folder


def read_folder(folder: str):
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as fh:
        config = json.load(fh)
    return config, load_file(os.path.join(folder, "model.safetensors"))


# A router's choice between two experts is not compared in bfloat16 where a change of the router's logits by this
# share of their size could turn it (see `segedra_plain.route`): what reaches a router in bfloat16 differs from the
# exact input by about a hundredth after a few layers, and whichever of the two experts an implementation then takes
# is right.  Such tokens are left out of the bfloat16 comparison; the float32 comparison leaves none out.
CLOSE_CALL = 0.05
MOST_CLOSE_CALLS = 0.5


class Expected(lapevik.Expected):
    """Exact logits, what bfloat16 storage alone costs, what float32 arithmetic alone costs (the plain implementation
    in float32: a sharp softmax makes more of a rounded score than the flat float32 limit allows), and the tokens
    whose routers made a close call."""

    def __init__(self, exact: np.ndarray, rounded: Optional[np.ndarray], single: Optional[np.ndarray], margins: np.ndarray) -> None:
        self.clear = margins >= CLOSE_CALL
        if self.clear.any():
            super().__init__(exact[self.clear], rounded[self.clear] if rounded is not None else None)
        self.exact = exact
        self.float32_error = float(np.abs(single.astype(np.float64) - exact.astype(np.float64)).max()) if single is not None else 0.0


def expected(folder: str, requests: Dict[str, List[int]], dtype: str) -> Dict[str, Expected]:
    config, weights = read_folder(folder)
    out = {}
    for rid, toks in requests.items():
        margins: list = []
        exact = segedra_plain.forward(weights, config, toks, torch.float64, margins=margins).to(torch.float32).numpy()
        least = torch.stack(margins).min(0).values.numpy() if margins else np.full(len(toks), np.inf)
        rounded = single = None
        if dtype == "bfloat16":
            rounded = segedra_plain.forward(weights, config, toks, torch.float64, rounded=True).to(torch.float32).numpy()
        else:
            single = segedra_plain.forward(weights, config, toks, torch.float32).numpy()
        out[rid] = Expected(exact, rounded, single, least)
    return out


def check(got: np.ndarray, want: Expected, dtype: str, what: str) -> None:
    assert got.shape == want.exact.shape, f"{what}: logits {got.shape}, expected {want.exact.shape}"
    assert not np.isnan(got).any(), f"{what}: missing or NaN logits"
    if dtype == "float32":
        err = np.abs(got.astype(np.float64) - want.exact.astype(np.float64)).max(axis=1)
        limit = max(lapevik.FLOAT32_LIMIT * float(np.abs(want.exact).max()), 4.0 * want.float32_error)
        assert err.max() <= limit, f"{what}: first position over the limit {int(np.argmax(err > limit))}, error {err.max():.3e} vs {limit:.3e}"
        return
    assert (~want.clear).sum() <= max(2, MOST_CLOSE_CALLS * want.clear.size), f"{what}: too many close calls for a comparison in bfloat16"
    if not want.clear.any():
        return
    clear = lapevik.Expected.__new__(lapevik.Expected)
    clear.exact, clear.rms, clear.max = want.exact[want.clear], want.rms, want.max
    lapevik.check(got[want.clear], clear, dtype, what + " (tokens without a close call of a router)")
