"""Without a GPU: the plain implementation's mechanisms against library routines and invariants, the configuration
and the plan of the Segedra architecture, and everything around the kernels (pages, windows, looped layers with caches
of their own, portions, mixed steps) with the kernels replaced by torch stand-ins."""

import math

import numpy as np
import pytest
import torch

from helpers import cpu_ops, segedra, traces
from plain import segedra_plain as sp

F64 = torch.float64


# ---- the plain implementation itself -------------------------------------------------------------------------- #
def test_norm_has_unit_mean_square_and_a_weight_around_zero():
    x = torch.randn(5, 24, dtype=F64) * 3
    y = sp.rms_norm(x, torch.zeros(24, dtype=F64), 0.0, one_plus=True)
    assert torch.allclose((y * y).mean(-1), torch.ones(5, dtype=F64))
    w = torch.randn(24, dtype=F64)
    assert torch.allclose(sp.rms_norm(x, w, 1e-6, one_plus=True), sp.rms_norm(x, w + 1, 1e-6, one_plus=False))
    tiny = torch.full((1, 4), 1e-4, dtype=F64)
    assert torch.allclose(sp.rms_norm(tiny, None, 1e-6, False), tiny / math.sqrt(1e-8 + 1e-6))  # eps inside the root


def test_rotation_depends_on_the_distance_only_and_leaves_the_rest():
    q, k = torch.randn(1, 1, 10, dtype=F64), torch.randn(1, 1, 10, dtype=F64)
    at = lambda x, p: sp.rotate_pairs(x, torch.tensor([p]), 100.0, 6)  # noqa: E731
    assert torch.allclose((at(q, 9) * at(k, 4)).sum(), (at(q, 25) * at(k, 20)).sum())
    assert torch.equal(at(q, 7)[..., 6:], q[..., 6:])
    assert torch.allclose(at(q, 0), q)
    # pair (0, 1) turns by the position itself: base^0 = 1
    x = torch.tensor([[[1.0, 0.0, 0.0, 0.0]]], dtype=F64)
    assert torch.allclose(sp.rotate_pairs(x, torch.tensor([2]), 50.0, 4)[0, 0, :2], torch.tensor([math.cos(2.0), math.sin(2.0)], dtype=F64))
    # and pair (2, 3) by position * base^(-2/4)
    x = torch.tensor([[[0.0, 0.0, 1.0, 0.0]]], dtype=F64)
    a = 3 * 50.0 ** -0.5
    assert torch.allclose(sp.rotate_pairs(x, torch.tensor([3]), 50.0, 4)[0, 0, 2:], torch.tensor([math.cos(a), math.sin(a)], dtype=F64))


def test_sink_is_one_more_term_of_the_denominator():
    scores = torch.randn(3, 6, dtype=F64)
    sink = torch.tensor(0.7, dtype=F64)
    w = sp.sink_softmax(scores, sink)
    full = torch.softmax(torch.cat([scores, sink.expand(3, 1)], -1), -1)
    assert torch.allclose(w, full[:, :-1]) and torch.all(w.sum(-1) < 1)
    assert torch.allclose(sp.sink_softmax(scores, None), torch.softmax(scores, -1))
    assert torch.allclose(sp.sink_softmax(scores, torch.tensor(-1e9, dtype=F64)), torch.softmax(scores, -1))


def _attention_tensors(width, m, seed=0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=F64)  # noqa: E731
    return {"q": r(m["heads"] * m["dim"], width), "k": r(m["kv_heads"] * m["dim"], width), "v": r(m["kv_heads"] * m["vdim"], width),
            "o": r(width, m["heads"] * m["vdim"]), "q.norm": r(m["heads"] * m["dim"]).abs() + 0.5, "k.norm": r(m["kv_heads"] * m["dim"]).abs() + 0.5,
            "sink": r(m["heads"])}


def test_attention_window_reads_the_query_and_size_minus_one_before_it():
    m = {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 6, "scale": 0.5, "mask": {"size": 4}, "rot": {"base": 100.0, "dims": 4}}
    t = _attention_tensors(10, m)
    h = torch.randn(12, 10, dtype=F64)
    base = sp.attention(h, t, m, 1e-6)
    moved = h.clone()
    moved[5] += 1.0  # token 5 is read by the queries 5 .. 8 and by no other
    out = sp.attention(moved, t, m, 1e-6)
    changed = (out - base).abs().max(-1).values > 1e-12
    assert changed.tolist() == [5 <= i <= 8 for i in range(12)]


def test_attention_is_the_unrolled_formula_for_one_query():
    m = {"heads": 4, "kv_heads": 2, "dim": 6, "vdim": 5, "scale": 0.7, "mask": {"size": 3}, "rot": {"base": 10.0, "dims": 6}}
    t = _attention_tensors(9, m, seed=3)
    h = torch.randn(7, 9, dtype=F64)
    got = sp.attention(h, t, m, 1e-5)
    i, eps = 6, 1e-5
    q_all, k_all = h @ t["q"].T, h @ t["k"].T
    q_all = q_all / torch.sqrt((q_all ** 2).mean(-1, keepdim=True) + eps) * t["q.norm"]  # over all heads at once
    k_all = k_all / torch.sqrt((k_all ** 2).mean(-1, keepdim=True) + eps) * t["k.norm"]
    v_all = (h @ t["v"].T).reshape(7, 2, 5)
    pos = torch.arange(7)
    q_all = sp.rotate_pairs(q_all.reshape(7, 4, 6), pos, 10.0, 6)
    k_all = sp.rotate_pairs(k_all.reshape(7, 2, 6), pos, 10.0, 6)
    heads = []
    for head in range(4):
        g = head // 2
        keys = [4, 5, 6]
        e = torch.stack([torch.exp(0.7 * (q_all[i, head] * k_all[j, g]).sum()) for j in keys])
        heads.append((e[:, None] * v_all[keys, g]).sum(0) / (e.sum() + torch.exp(t["sink"][head])))
    assert torch.allclose(got[i], torch.cat(heads) @ t["o"].T)


def test_router_correction_changes_the_choice_and_not_the_weights():
    h = torch.randn(50, 12, dtype=F64)
    t = {"router": torch.randn(6, 12, dtype=F64)}
    chosen0, w0 = sp.route(h, t, 2, 2.5)
    s = torch.softmax(h @ t["router"].T, -1)
    assert torch.equal(chosen0, torch.topk(s, 2, -1).indices)
    assert torch.allclose(w0, 2.5 * torch.gather(s, 1, chosen0))  # not renormalised
    t["correction"] = torch.tensor([5.0, 0, 0, 0, 0, -5.0], dtype=F64)
    chosen1, w1 = sp.route(h, t, 2, 2.5)
    assert torch.all(chosen1[:, 0] == 0) and not torch.any(chosen1 == 5)
    assert torch.allclose(w1, 2.5 * torch.gather(s, 1, chosen1))


def test_expert_clamps_gate_from_above_and_up_on_both_sides():
    eye = torch.eye(3, dtype=F64)
    h = torch.tensor([[-4.0, 0.3, 9.0]], dtype=F64)
    got = sp.expert(h, eye, eye, eye, 1.0)
    g = torch.tensor([-4.0, 0.3, 1.0], dtype=F64)
    u = torch.tensor([-1.0, 0.3, 1.0], dtype=F64)
    assert torch.allclose(got, (g * torch.sigmoid(1.702 * g) * (u + 1))[None])


def test_streams_with_unit_coefficients_are_the_plain_residual():
    x, y = torch.randn(1, 4, 6, dtype=F64), torch.randn(4, 6, dtype=F64)
    one = torch.ones(1, dtype=F64)
    assert torch.allclose(sp.write_streams(x, y, torch.ones(1, 1, dtype=F64), one), x + y[None])
    assert torch.allclose(sp.read_streams(x, one), x[0])
    xs = torch.randn(3, 4, 6, dtype=F64)
    mix = torch.randn(3, 3, dtype=F64)
    new = sp.write_streams(xs, y, mix, torch.tensor([1.0, 2.0, 3.0], dtype=F64))
    assert torch.allclose(new[2], mix[0, 2] * xs[0] + mix[1, 2] * xs[1] + mix[2, 2] * xs[2] + 3 * y)  # [from, to]


def test_loop_order():
    config = {"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 3}}
    assert sp.layer_order(config) == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert sp.layer_order({"layers": [0] * 3}) == [0, 1, 2]
    assert sp.layer_order({"layers": [0] * 3, "loop": {"start": 2, "stop": 2, "times": 4}}) == [0, 1, 2]


def test_a_window_one_key_off_or_a_sink_left_out_would_show():
    """tiny_t's softmax is sharp: the plain implementation with its windows one key longer or shorter, or without its
    sinks, differs from the true one by far more than any limit of the comparisons with the engine."""
    import copy

    config = segedra.get("tiny_t")
    weights = segedra.draw_weights(config, 5)
    toks = traces.random_tokens(99, 200, config["vocab"])
    exact = sp.forward(weights, config, toks)
    for off in (-1, 1):
        other = copy.deepcopy(config)
        for layer in other["layers"]:
            if "mask" in layer["mixer"]:
                layer["mixer"]["mask"]["size"] += off
        assert (sp.forward(weights, other, toks) - exact).abs().max() > 1e-2 * exact.abs().max()
    no_sink = {k: v for k, v in weights.items() if not k.endswith("mix.sink")}
    assert (sp.forward(no_sink, config, toks) - exact).abs().max() > 1e-2 * exact.abs().max()


# ---- configuration and plan ------------------------------------------------------------------------------------- #
def test_config_is_strict_and_the_plan_names_the_folder_s_tensors():
    from cwm_amd.config import ConfigError, parse_config
    from cwm_amd.models.model import Model
    from cwm_amd.parts.base import PagedKVSpec

    for name in segedra.ALL:
        config = segedra.get(name)
        arch, typed = parse_config(config)
        assert arch.name == "Segedra"
        model = Model(arch.build_plan(typed))
        weights = segedra.draw_weights(config, 1)
        specs = model.tensor_specs()
        assert set(specs) == set(weights)
        assert all(tuple(weights[k].shape) == tuple(specs[k].shape) for k in specs)
        order = sp.layer_order(config)
        assert [call.layer for call in model.run_order] == order
        assert len(model.cache_specs) == len(order)  # every pass of a looped layer keeps a cache of its own
        for spec, index in zip(model.cache_specs, order):
            m = config["layers"][index]["mixer"]
            assert isinstance(spec, PagedKVSpec) and spec.n_kv_heads == m["kv_heads"] and spec.head_dim >= max(m["dim"], m["vdim"])
            assert spec.window == (m["mask"]["size"] if "mask" in m else None)
    bad = segedra.get("tiny_s")
    bad["layers"][0]["mixer"]["windows"] = 3
    with pytest.raises(ConfigError, match="windows"):
        parse_config(bad)
    bad = segedra.get("tiny_s")
    bad["loop"]["stop"] = 9
    with pytest.raises(ConfigError, match="loop"):
        parse_config(bad)
    bad = segedra.get("tiny_t")
    bad["layers"][1]["mlp"] = {"kind": "dense", "ff": 8, "router": {"experts": 2, "top": 1}}
    with pytest.raises(ConfigError):
        parse_config(bad)


# ---- everything around the kernels ----------------------------------------------------------------------------- #
LENGTHS = {"tiny_s": [1, 6, 21, 40], "tiny_t": [9, 33, 2, 17, 26], "tiny_u": [30, 12, 45]}


@pytest.mark.parametrize("name", list(segedra.ALL))
@pytest.mark.parametrize("regime", ["whole", "tail", "portions", "mixed"])
def test_regimes_against_plain(tmp_path, monkeypatch, name, regime):
    """Pages that are freed (also by the windows) and used again, portions down to two tokens, unequal requests side
    by side: with torch in the kernels' place every difference is a fault of the descriptor, the tables or the plan."""
    from cwm_amd.replay import Replayer

    cpu_ops.install(monkeypatch)
    folder = segedra.make_folder(tmp_path, name, seed=3)
    vocab = segedra.get(name)["vocab"]
    requests = {f"r{i}": traces.random_tokens(11 * i + len(name), n, vocab) for i, n in enumerate(LENGTHS[name])}
    steps = {"whole": traces.whole, "tail": lambda r: traces.tail_one_by_one(r, tail=8), "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, max_live=2, decode_tail=5)}[regime](requests)
    rep = Replayer(folder, "float32", traces.max_live_tokens(steps), device="cpu", page_size=4 if regime == "mixed" else 16,
                   max_requests=2 if regime == "mixed" else 4, poison_freed_pages=True)
    outputs = traces.run_in_process(rep, steps)
    got = traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab)
    want = segedra.expected(folder, requests, "float32")
    for rid in requests:
        assert not np.isnan(got[rid]).any(), f"{rid}: missing or NaN logits"
        np.testing.assert_allclose(got[rid], want[rid].exact, rtol=2e-3, atol=2e-4 * float(np.abs(want[rid].exact).max()), err_msg=f"{name} {regime} {rid}")
    assert rep.manager.live_requests() == []
    assert all(f == g.pool.num_pages for f, g in zip(rep.manager.free_pages(), rep.manager.groups))
