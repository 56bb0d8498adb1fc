"""Tiny configurations of the Lapevik architecture with weights drawn so that every mechanism matters, the writer
of their model folders, and the plain implementation's logits for them.

The sizes differ from one another wherever two could be equal (heads, head size, state rows, groups, ranks, the
rotated part and how much of it turns, experts and how many a token uses, taps, norm groups), and layers come
with and without a feed-forward."""

from __future__ import annotations

import copy
import json
import os
from typing import Dict, List, Optional

import numpy as np
import torch

from plain import lapevik_plain


def _moe(ff: int, experts: int, top: int) -> dict:
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def _ssm(heads, vdim, state, groups, norm_groups, conv, kind="mamba2", mlp=None) -> dict:
    return {"type": kind, "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}, "mlp": mlp}


def _attn(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base, dims, mlp=None) -> dict:
    return {
        "type": "latent_attention",
        "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
                  "rot": {"base": base, "dims": dims}},
        "mlp": mlp,
    }


# a cached row of 8 + 40 = 48 elements: the matrix-core attention in bfloat16
TINY_P = {
    "architecture": "Lapevik", "vocab": 211, "width": 64, "norm": {"eps": 1e-5, "groups": 2},
    "layers": [
        _ssm(3, 16, 24, 1, 3, 3, mlp=_moe(40, 4, 2)),
        _attn(3, 24, 8, 20, 40, 32, 0.2, 10000.0, 8),
        _ssm(4, 8, 16, 2, 1, 4, kind="mamba2_2", mlp=_moe(24, 5, 1)),
    ],
}
# rows of 12 + 30 = 42 (the plain attention kernel in both types; 8 of the 12 rotated elements turn) and of 16 + 64 = 80
TINY_Q = {
    "architecture": "Lapevik", "vocab": 97, "width": 96, "norm": {"eps": 1e-6, "groups": 1},
    "layers": [
        _attn(5, 12, 12, 28, 30, 20, 0.3, 500.0, 8, mlp=_moe(36, 3, 3)),
        _ssm(2, 40, 70, 2, 4, 2),
        _attn(2, 32, 16, 16, 64, 48, 0.25, 300000.0, 16, mlp=_moe(16, 6, 2)),
    ],
}
# a sharp softmax (large scale) over long sequences: one key far back, or just behind a page border, carries a token's
# result; a slow state (small decay) that remembers the sequence's start
TINY_R = {
    "architecture": "Lapevik", "vocab": 131, "width": 48, "norm": {"eps": 1e-5, "groups": 3},
    "layers": [
        _attn(2, 16, 16, 24, 16, 24, 2.5, 1000.0, 16, mlp=_moe(20, 2, 1)),
        _ssm(2, 12, 20, 1, 2, 5, mlp=None),
    ],
}

# wider, so that a prompt of some hundred tokens takes the kernels' shapes for many rows (library products, the
# attention's long-portion kernel on a row of 128, segments of the recurrence, the grouped product through LDS)
MEDIUM = {
    "architecture": "Lapevik", "vocab": 300, "width": 256, "norm": {"eps": 1e-5, "groups": 4},
    "layers": [
        _ssm(8, 32, 64, 2, 2, 4, mlp=_moe(128, 2, 1)),
        _attn(4, 32, 32, 64, 96, 64, 0.125, 10000.0, 32, mlp=_moe(64, 3, 2)),
    ],
}

ALL = {"tiny_p": TINY_P, "tiny_q": TINY_Q, "tiny_r": TINY_R}


def get(name: str) -> dict:
    return copy.deepcopy(ALL[name])


def draw_weights(config: dict, seed: int) -> Dict[str, torch.Tensor]:
    """bfloat16 tensors by name.  Matrices N(0, 1 / fan-in); norm weights, the shift and the skip in ranges where they
    do something; decays slow enough that the state carries far; a router with clear choices."""
    gen = torch.Generator().manual_seed(seed)
    normal = lambda *shape, std=1.0: torch.randn(*shape, generator=gen) * std  # noqa: E731
    uniform = lambda lo, hi, *shape: torch.rand(*shape, generator=gen) * (hi - lo) + lo  # noqa: E731
    matrix = lambda out, inp: normal(out, inp, std=inp ** -0.5)  # noqa: E731
    width, vocab = config["width"], config["vocab"]
    w = {"embed": normal(vocab, width), "embed.norm": uniform(0.5, 1.5, width), "final.norm": uniform(0.5, 1.5, width)}
    for i, layer in enumerate(config["layers"]):
        m, p = layer["mixer"], f"l{i}."
        w[p + "shift"] = uniform(0.0, 1.0, width)
        w[p + "norm1"] = uniform(0.5, 1.5, width)
        if lapevik_plain.mixer_kind(layer["type"]) == "mamba2":
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            w[p + "mix.in"] = matrix(2 * inner + 2 * gn + m["heads"], width)
            w[p + "mix.conv"] = normal(inner + 2 * gn, m["conv"], std=0.5)
            w[p + "mix.conv.b"] = normal(inner + 2 * gn, std=0.2)
            w[p + "mix.dt_bias"] = uniform(-2.0, 0.0, m["heads"])
            w[p + "mix.A_log"] = uniform(-4.0, -1.0, m["heads"])
            w[p + "mix.D"] = normal(m["heads"], std=0.5) + 1.0
            w[p + "mix.norm"] = uniform(0.5, 1.5, inner)
            w[p + "mix.o"] = matrix(width, inner)
        else:
            h = m["heads"]
            w[p + "mix.dq"] = matrix(m["q_rank"], width)
            w[p + "mix.dq.norm"] = uniform(0.5, 1.5, m["q_rank"])
            w[p + "mix.uq"] = matrix(h * (m["dim"] + m["rot_dim"]), m["q_rank"])
            w[p + "mix.dkv"] = matrix(m["kv_rank"] + m["rot_dim"], width)
            w[p + "mix.dkv.norm"] = uniform(0.5, 1.5, m["kv_rank"])
            w[p + "mix.uk"] = matrix(h * m["dim"], m["kv_rank"])
            w[p + "mix.uv"] = matrix(h * m["vdim"], m["kv_rank"])
            w[p + "mix.g"] = matrix(h * m["vdim"], width)
            w[p + "mix.o"] = matrix(width, h * m["vdim"])
        if layer["mlp"] is not None:
            ff, experts = layer["mlp"]["expert"]["ff"], layer["mlp"]["router"]["experts"]
            w[p + "norm2"] = uniform(0.5, 1.5, width)
            w[p + "mlp.router"] = normal(experts, width, std=0.5)
            for e in range(experts):
                w[p + f"mlp.e{e}.gate"] = matrix(ff, width)
                w[p + f"mlp.e{e}.up"] = matrix(ff, width)
                w[p + f"mlp.e{e}.down"] = matrix(width, ff)
    return {k: v.to(torch.bfloat16).contiguous() for k, v in w.items()}


def make_folder(root, name: str, seed: int = 1, config: Optional[dict] = None) -> str:
    from safetensors.torch import save_file

    config = config or get(name)
    folder = os.path.join(str(root), f"{name}_{seed}")
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(config, fh)
    save_file(draw_weights(config, seed), os.path.join(folder, "model.safetensors"))
    return folder


def read_folder(folder: str):
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as fh:
        config = json.load(fh)
    return config, load_file(os.path.join(folder, "model.safetensors"))


class Expected:
    """Exact logits of a request (float64 arithmetic on the stored weights) and what bfloat16 storage alone costs."""

    def __init__(self, exact: np.ndarray, rounded: Optional[np.ndarray]) -> None:
        self.exact = exact
        if rounded is not None:
            diff = rounded.astype(np.float64) - exact.astype(np.float64)
            self.rms = float(np.sqrt((diff * diff).mean()))
            self.max = float(np.abs(diff).max())


def expected(folder: str, requests: Dict[str, List[int]], dtype: str) -> Dict[str, Expected]:
    config, weights = read_folder(folder)
    out = {}
    for rid, toks in requests.items():
        exact = lapevik_plain.forward(weights, config, toks, torch.float64).to(torch.float32).numpy()
        rounded = None
        if dtype == "bfloat16":
            rounded = lapevik_plain.forward(weights, config, toks, torch.float64, rounded=True).to(torch.float32).numpy()
        out[rid] = Expected(exact, rounded)
    return out


FLOAT32_LIMIT = 3e-5  # of the request's largest logit: float32 sums in another order, nothing else
BF16_RMS_RATIO = 2.0  # of what the plain implementation's own bfloat16 run loses
BF16_MAX_RATIO = 4.0


def check(got: np.ndarray, want: Expected, dtype: str, what: str) -> None:
    assert got.shape == want.exact.shape, f"{what}: logits {got.shape}, expected {want.exact.shape}"
    assert not np.isnan(got).any(), f"{what}: missing or NaN logits"
    diff = got.astype(np.float64) - want.exact.astype(np.float64)
    err = np.abs(diff).max(axis=1)
    if dtype == "float32":
        limit = FLOAT32_LIMIT * float(np.abs(want.exact).max())
        assert err.max() <= limit, f"{what}: first position over the limit {int(np.argmax(err > limit))}, error {err.max():.3e} vs {limit:.3e}"
        return
    rms = float(np.sqrt((diff * diff).mean()))
    assert err.max() <= BF16_MAX_RATIO * want.max, (
        f"{what}: first position over the limit {int(np.argmax(err > BF16_MAX_RATIO * want.max))}, error {err.max():.3e} is "
        f"{err.max() / want.max:.2f} times what bfloat16 storage costs"
    )
    assert rms <= BF16_RMS_RATIO * want.rms, f"{what}: root-mean-square error {rms:.3e} is {rms / want.rms:.2f} times what bfloat16 storage costs"
