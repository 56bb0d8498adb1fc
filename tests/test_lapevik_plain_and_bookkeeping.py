"""Without a GPU: the plain implementation's mechanisms against library routines and invariants, the
configuration and the plan of the Lapevik architecture, and everything around the kernels (state slots, pages,
portions, mixed steps) with the kernels replaced by torch stand-ins."""

import numpy as np
import pytest
import torch

from helpers import cpu_ops, lapevik, traces
from plain import lapevik_plain as lp


# ---- the plain implementation itself -------------------------------------------------------------------------- #
def test_group_norm_parts_have_unit_mean_square():
    x = torch.randn(5, 24, dtype=torch.float64) * 3
    y = lp.group_rms_norm(x, torch.ones(24, dtype=torch.float64), 4, 0.0)
    assert torch.allclose((y.reshape(5, 4, 6) ** 2).mean(-1), torch.ones(5, 4, dtype=torch.float64))
    one = lp.group_rms_norm(x, torch.ones(24, dtype=torch.float64), 1, 1e-6)
    assert torch.allclose(one, x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-6))


def test_token_shift_ends():
    x = torch.randn(4, 6, dtype=torch.float64)
    assert torch.equal(lp.token_shift(x, torch.zeros(6, dtype=torch.float64)), x)
    shifted = lp.token_shift(x, torch.ones(6, dtype=torch.float64))
    assert torch.allclose(shifted[1:], x[:-1]) and torch.all(shifted[0] == 0)


def test_causal_conv_is_the_library_convolution():
    u, w, b = torch.randn(9, 5, dtype=torch.float64), torch.randn(5, 4, dtype=torch.float64), torch.randn(5, dtype=torch.float64)
    padded = torch.nn.functional.pad(u.T[None], (3, 0))
    want = torch.nn.functional.conv1d(padded, w[:, None, :], b, groups=5)[0].T
    assert torch.allclose(lp.causal_conv(u, w, b), want)


def test_rotation_depends_on_the_distance_only():
    q, k = torch.randn(1, 8, dtype=torch.float64), torch.randn(1, 8, dtype=torch.float64)
    at = lambda x, p: lp.rotate_pairs(x, torch.tensor([p]), 100.0, 6)  # noqa: E731
    assert torch.allclose((at(q, 9) * at(k, 4)).sum(), (at(q, 25) * at(k, 20)).sum())
    assert torch.equal(at(q, 7)[..., 6:], q[..., 6:])  # beyond the rotated elements nothing turns
    assert torch.allclose(at(q, 0), q)


def test_state_space_is_the_unrolled_sum():
    """With a decay of its own per step, y_t = sum_(s<=t) (prod_(s<r<=t) a_r) dt_s (C_t . B_s) x_s + D x_t."""
    torch.manual_seed(0)
    heads, vdim, state, n = 2, 3, 4, 6
    inner, width = heads * vdim, 10
    t = {
        "in": torch.randn(2 * inner + 2 * state + heads, width, dtype=torch.float64) * 0.3,
        "conv": torch.zeros(inner + 2 * state, 2, dtype=torch.float64), "conv.b": torch.zeros(inner + 2 * state, dtype=torch.float64),
        "dt_bias": torch.randn(heads, dtype=torch.float64), "A_log": torch.randn(heads, dtype=torch.float64), "D": torch.randn(heads, dtype=torch.float64),
        "norm": torch.ones(inner, dtype=torch.float64), "o": torch.eye(inner, dtype=torch.float64),
    }
    t["conv"][:, 1] = 1.0  # the convolution passes the current input
    s = torch.randn(n, width, dtype=torch.float64)
    got = lp.state_space(s, t, heads, vdim, state, 1, 1, 0.0)
    u = s @ t["in"].T
    z, xs, b, c, dt = u[:, :inner], lp.silu(u[:, inner : 2 * inner]), lp.silu(u[:, 2 * inner : 2 * inner + state]), lp.silu(u[:, 2 * inner + state : 2 * inner + 2 * state]), u[:, 2 * inner + 2 * state :]
    dt = torch.log1p(torch.exp(dt + t["dt_bias"]))
    a = torch.exp(-torch.exp(t["A_log"]) * dt)
    y = torch.zeros(n, heads, vdim, dtype=torch.float64)
    for h in range(heads):
        x = xs[:, h * vdim : (h + 1) * vdim]
        for i in range(n):
            for j in range(i + 1):
                y[i, h] += torch.prod(a[j + 1 : i + 1, h]) * dt[j, h] * (c[i] @ b[j]) * x[j]
            y[i, h] += t["D"][h] * x[i]
    want = lp.group_rms_norm(y.reshape(n, inner) * lp.silu(z), t["norm"], 1, 0.0)
    assert torch.allclose(got, want)


def test_latent_attention_is_attention_over_expanded_keys():
    torch.manual_seed(1)
    heads, dim, rot, vdim, kr, qr, width, n = 2, 4, 2, 3, 5, 6, 7, 5
    t = {k: torch.randn(*shape, dtype=torch.float64) for k, shape in {
        "dq": (qr, width), "dq.norm": (qr,), "uq": (heads * (dim + rot), qr), "dkv": (kr + rot, width), "dkv.norm": (kr,),
        "uk": (heads * dim, kr), "uv": (heads * vdim, kr), "g": (heads * vdim, width), "o": (width, heads * vdim)}.items()}
    s = torch.randn(n, width, dtype=torch.float64)
    got = lp.latent_attention(s, t, heads, dim, rot, vdim, kr, 0.4, 50.0, 2, 1e-5)
    pos = torch.arange(n)
    cq = lp.group_rms_norm(s @ t["dq"].T, t["dq.norm"], 1, 1e-5)
    q = (cq @ t["uq"].T).reshape(n, heads, dim + rot)
    down = s @ t["dkv"].T
    c = lp.group_rms_norm(down[:, :kr], t["dkv.norm"], 1, 1e-5)
    kr_rot = lp.rotate_pairs(down[:, kr:], pos, 50.0, 2)
    out = torch.zeros(n, heads, vdim, dtype=torch.float64)
    for h in range(heads):
        k = torch.cat([c @ t["uk"][h * dim : (h + 1) * dim].T, kr_rot], -1)
        qh = torch.cat([q[:, h, :dim], lp.rotate_pairs(q[:, h, dim:], pos, 50.0, 2)], -1)
        v = c @ t["uv"][h * vdim : (h + 1) * vdim].T
        out[:, h] = torch.nn.functional.scaled_dot_product_attention(qh[None], k[None], v[None], is_causal=True, scale=0.4)[0]
    want = (out.reshape(n, -1) * torch.sigmoid(s @ t["g"].T)) @ t["o"].T
    assert torch.allclose(got, want)


def test_routed_experts_ends():
    torch.manual_seed(2)
    t = {"router": torch.randn(3, 6, dtype=torch.float64)}
    for e in range(3):
        t[f"e{e}.gate"], t[f"e{e}.up"], t[f"e{e}.down"] = torch.randn(4, 6, dtype=torch.float64), torch.randn(4, 6, dtype=torch.float64), torch.randn(6, 4, dtype=torch.float64)
    x = torch.randn(5, 6, dtype=torch.float64)
    each = [(lp.silu(x @ t[f"e{e}.gate"].T) * (x @ t[f"e{e}.up"].T)) @ t[f"e{e}.down"].T for e in range(3)]
    logits = x @ t["router"].T
    all_of_them = sum(torch.softmax(logits, -1)[:, e : e + 1] * each[e] for e in range(3))
    assert torch.allclose(lp.routed_experts(x, t, 3, 3), all_of_them)
    best = logits.argmax(-1)
    assert torch.allclose(lp.routed_experts(x, t, 3, 1), torch.stack([each[int(best[i])][i] for i in range(5)]))


# ---- configuration and plan ------------------------------------------------------------------------------------ #
def test_configuration_is_strict_and_kinds_take_suffixes():
    from cwm_amd.config import ConfigError, parse_config

    arch, cfg = parse_config(lapevik.get("tiny_p"))
    assert arch.name == "Lapevik" and [type(layer.mixer_config()).__name__ for layer in cfg.layers] == ["StateSpaceConfig", "LatentAttentionConfig", "StateSpaceConfig"]
    assert cfg.layers[1].mlp is None and cfg.layers[2].mlp.router.top == 1
    for breakage, key in (
        (lambda c: c["layers"][0]["mixer"].update(window=4), "window"),
        (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
        (lambda c: c["layers"][0].update(type="conv_mixer"), "conv_mixer"),
        (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "dense"),
        (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top"),
        (lambda c: c["norm"].update(groups=5), "groups"),
    ):
        broken = lapevik.get("tiny_p")
        breakage(broken)
        with pytest.raises(ConfigError, match=key):
            parse_config(broken)


def test_plan_names_the_folder_tensors_and_states():
    from cwm_amd.config import parse_config
    from cwm_amd.models import Model
    from cwm_amd.parts import PagedKVSpec, StateSpec

    for name in lapevik.ALL:
        config = lapevik.get(name)
        arch, cfg = parse_config(config)
        model = Model(arch.build_plan(cfg))
        weights = lapevik.draw_weights(config, 0)
        specs = model.tensor_specs()
        assert set(specs) == set(weights)
        assert all(tuple(weights[k].shape) == tuple(specs[k].shape) for k in specs)
        # a state for every layer's shift, one for every state-space mixer, pages of one row a token for every attention
        kinds = [type(s).__name__ for s in model.cache_specs]
        assert kinds.count("StateSpec") == len(config["layers"]) + sum(lp.mixer_kind(l["type"]) == "mamba2" for l in config["layers"])
        for layer, slots in zip(config["layers"], model.cache_slots):
            spec = model.cache_specs[slots[1]]
            m = layer["mixer"]
            if lp.mixer_kind(layer["type"]) == "mamba2":
                # every head's state (the kernel may pad it) and the convolution's last inputs
                assert isinstance(spec, StateSpec) and spec.shape[0] >= m["heads"] * m["state"] * m["vdim"] + (m["conv"] - 1) * (m["heads"] * m["vdim"] + 2 * m["groups"] * m["state"])
            else:
                assert isinstance(spec, PagedKVSpec) and spec.n_kv_heads == 1 and spec.head_dim == m["kv_rank"] + m["rot_dim"] and spec.window is None


# ---- everything around the kernels ----------------------------------------------------------------------------- #
LENGTHS = {"tiny_p": [1, 6, 21, 40], "tiny_q": [9, 33, 2, 17, 26], "tiny_r": [30, 12, 45]}


@pytest.mark.parametrize("name", list(lapevik.ALL))
@pytest.mark.parametrize("regime", ["whole", "tail", "portions", "mixed"])
def test_regimes_against_plain(tmp_path, monkeypatch, name, regime):
    """State slots and pages that are freed and used again, portions down to two tokens, unequal requests side by
    side: with torch in the kernels' place every difference is a fault of the descriptor, the tables or the state."""
    from cwm_amd.replay import Replayer

    cpu_ops.install(monkeypatch)
    folder = lapevik.make_folder(tmp_path, name, seed=3)
    vocab = lapevik.get(name)["vocab"]
    requests = {f"r{i}": traces.random_tokens(11 * i + len(name), n, vocab) for i, n in enumerate(LENGTHS[name])}
    steps = {"whole": traces.whole, "tail": lambda r: traces.tail_one_by_one(r, tail=8), "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, max_live=2, decode_tail=5)}[regime](requests)
    rep = Replayer(folder, "float32", traces.max_live_tokens(steps), device="cpu", page_size=4 if regime == "mixed" else 16,
                   max_requests=2 if regime == "mixed" else 4, poison_freed_pages=True)
    outputs = traces.run_in_process(rep, steps)
    got = traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab)
    want = lapevik.expected(folder, requests, "float32")
    for rid in requests:
        assert not np.isnan(got[rid]).any(), f"{rid}: missing or NaN logits"
        np.testing.assert_allclose(got[rid], want[rid].exact, rtol=2e-3, atol=2e-4 * float(np.abs(want[rid].exact).max()), err_msg=f"{name} {regime} {rid}")
    assert rep.manager.live_requests() == []
    assert all(f == g.pool.num_pages for f, g in zip(rep.manager.free_pages(), rep.manager.groups))
