"""The Segedra architecture on the GPU against the plain implementation.

First each new kernel alone against plain PyTorch in float32 (streams with their norm, the activation, the norm
over whole projections with rotation and cache write, the router over all experts, the clamped gated product, the
sink in every path of both attention kernels); then models: every regime of the replay driver in both types with pages
that are used again; single layers that leave one mechanism nearly alone; a sharp attention whose tokens hang on single
keys far back and at a window's edge; first tokens and long decoding; looped layers; decode steps replayed from
graphs; and greedy generation through the engine, the command line and `bin/trace_run`."""

import json
import os
import subprocess
import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from helpers import cache_layout, segedra, traces
from plain import segedra_plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def rnd(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g) * scale


def tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


# ---- kernels ----------------------------------------------------------------------------------------------------- #
@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("streams,dim,parts", [(1, 40, 1), (2, 256, 3), (3, 120, 1), (4, 1000, 2), (8, 7, 1), (5, 6144, 1)])
def test_stream_mix_norm(out_dtype, streams, dim, parts):
    from cwm_amd import ops

    n = 9
    x = rnd((n, streams, dim), 1, 2.0)
    y = rnd((parts, n, dim), 2) if parts > 1 else rnd((n, dim), 2)
    mix, b, a, w = rnd((streams, streams), 3), rnd((streams,), 4), rnd((streams,), 5), rnd((dim,), 6) + 1
    ysum = y.sum(0) if parts > 1 else y
    new = torch.einsum("st,nsd->ntd", mix.double(), x.double()) + b.double()[None, :, None] * ysum.double()[:, None, :]
    u = (a.double()[None, :, None] * new).sum(1)
    want = u / torch.sqrt((u * u).mean(-1, keepdim=True) + 1e-5) * w.double()
    xd = x.reshape(n, streams * dim).to(DEV).contiguous()
    # chosen rows first: the streams stay as they are
    rows = torch.tensor([7, 0, 3], dtype=torch.int32, device=DEV)
    got = ops.stream_mix_norm(xd, streams, y.to(DEV), mix.to(DEV), b.to(DEV), a.to(DEV), w.to(DEV), 1e-5, out_dtype, rows)
    assert torch.equal(xd.cpu(), x.reshape(n, -1))
    torch.testing.assert_close(got.cpu().double(), want[[7, 0, 3]], **tol(out_dtype))
    got = ops.stream_mix_norm(xd, streams, y.to(DEV), mix.to(DEV), b.to(DEV), a.to(DEV), w.to(DEV), 1e-5, out_dtype)
    torch.testing.assert_close(got.cpu().double(), want, **tol(out_dtype))
    torch.testing.assert_close(xd.cpu().double().view(n, streams, dim), new, rtol=1e-5, atol=1e-5)
    # nothing pending, no coefficients: the norm of the sum of the streams
    total = new.sum(1)
    want = total / torch.sqrt((total * total).mean(-1, keepdim=True) + 1e-5) * w.double()
    got = ops.stream_mix_norm(xd, streams, None, None, None, None, w.to(DEV), 1e-5, torch.float32)
    torch.testing.assert_close(got.cpu().double(), want, rtol=2e-5, atol=2e-5)
    # a pending result without coefficients is the plain sum into every stream
    y16 = rnd((n, dim), 8).to(torch.bfloat16)
    before = xd.clone()
    ops.stream_mix_norm(xd, streams, y16.to(DEV), None, None, None, w.to(DEV), 1e-5, torch.float32)
    torch.testing.assert_close(xd.cpu().view(n, streams, dim), before.cpu().view(n, streams, dim) + y16.float()[:, None, :], rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("streams,dim", [(4, 128), (1, 50), (3, 72)])
def test_stream_mix_norm_adds_up_a_weighted_sum_of_rows_itself(streams, dim):
    """The experts' rows of every (token, choice) pair and the router's weights as the pending result: the same bits as
    from the rows added up beforehand."""
    from cwm_amd import ops

    tokens, experts, top = 21, 5, 3
    g = torch.Generator().manual_seed(2)
    chosen = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(tokens)]).to(torch.int32)
    groups = ops.group_by_expert(chosen.to(DEV), experts)
    rows = rnd((groups.n_tiles * 16, dim), 3).to(DEV)
    weights = torch.rand((tokens, top), generator=g).to(DEV)
    routed = ops.RoutedSum(rows, groups, weights)
    mix, b, a, w = rnd((streams, streams), 3).to(DEV), rnd((streams,), 4).to(DEV), rnd((streams,), 5).to(DEV), (rnd((dim,), 6) + 1).to(DEV)
    x1 = rnd((tokens, streams * dim), 7).to(DEV)
    x2 = x1.clone()
    got = ops.stream_mix_norm(x1, streams, routed, mix, b, a, w, 1e-5, torch.float32)
    want = ops.stream_mix_norm(x2, streams, routed.combine(), mix, b, a, w, 1e-5, torch.float32)
    assert torch.equal(got, want) and torch.equal(x1, x2)
    picked = torch.tensor([20, 4], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.stream_mix_norm(x1, streams, routed, mix, b, a, w, 1e-5, torch.bfloat16, picked),
                       ops.stream_mix_norm(x2, streams, routed.combine(), mix, b, a, w, 1e-5, torch.bfloat16, picked))


def test_embedding_starts_every_stream():
    from cwm_amd import ops

    table = rnd((50, 24), 1).to(torch.bfloat16)
    tokens = torch.tensor([3, 49, 0, 3], dtype=torch.int32)
    got = ops.embedding_streams(tokens.to(DEV), table.to(DEV), 3, 2.5).cpu()
    want = (table[tokens.long()].float() * 2.5)[:, None, :].expand(4, 3, 24).reshape(4, 72)
    assert torch.equal(got, want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["relu2", "relu", "gelu_tanh", "silu"])
def test_act_rows(dtype, kind):
    from cwm_amd import ops

    x = rnd((13, 77), 3, 2.0).to(dtype)
    f = {"relu2": lambda z: torch.relu(z) ** 2, "relu": torch.relu, "silu": torch.nn.functional.silu,
         "gelu_tanh": lambda z: torch.nn.functional.gelu(z, approximate="tanh")}[kind]
    torch.testing.assert_close(ops.act_rows(x.to(DEV), kind, dtype).cpu().double(), f(x.double()), **tol(dtype))
    parts = rnd((3, 13, 77), 4)
    torch.testing.assert_close(ops.act_rows(parts.to(DEV), kind, dtype).cpu().double(), f(parts.double().sum(0)), **tol(dtype))


@pytest.mark.parametrize("src_dtype,dtype", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16), (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("n_q,n_kv,qk,vd,hd,rot,page_size,norm", [
    (4, 2, 12, 20, 32, 8, 8, True), (3, 1, 10, 6, 16, 4, 8, True), (3, 3, 64, 64, 64, 64, 16, True), (6, 1, 80, 48, 80, 40, 5, True), (2, 2, 16, 16, 16, 0, 4, False), (5, 5, 24, 8, 32, 24, 32, True),
])
def test_qk_norm_rope_write(src_dtype, dtype, n_q, n_kv, qk, vd, hd, rot, page_size, norm):
    """A fresh prompt, a continued portion and a decoded token in one call, from the projection itself and from partial
    sums: the queries, and the keys and values where the block table says, padded with zeros to the cached head."""
    from cwm_amd import ops

    lens_old, lens_new = [0, 37, 70], [29, 21, 1]
    width = (n_q + n_kv) * qk + n_kv * vd
    n = sum(lens_new)
    positions = torch.cat([torch.arange(a, a + b) for a, b in zip(lens_old, lens_new)]).to(torch.int32)
    seq_of = torch.cat([torch.full((b,), i) for i, b in enumerate(lens_new)]).to(torch.int32)
    pages_per = [(a + b + page_size - 1) // page_size for a, b in zip(lens_old, lens_new)]
    perm = torch.randperm(sum(pages_per) + 2, generator=torch.Generator().manual_seed(1)).tolist()
    table = torch.full((3, max(pages_per)), -1, dtype=torch.int32)
    for b, count in enumerate(pages_per):
        for lp in range(count):
            table[b, lp] = perm.pop()
    qw, kw = (rnd((n_q * qk,), 5).abs() + 0.5, rnd((n_kv * qk,), 6).abs() + 0.5) if norm else (None, None)
    inv_freq = None
    if rot:
        inv_freq = torch.zeros(hd // 2)
        inv_freq[: rot // 2] = torch.tensor([300.0 ** (-2.0 * i / rot) for i in range(rot // 2)])
    for parts in (1, 3):
        if parts > 1 and src_dtype != torch.float32:
            continue
        src = rnd((parts, n, width), 7 + parts).to(src_dtype) if parts > 1 else rnd((n, width), 7).to(src_dtype)
        full = (src.double().sum(0) if parts > 1 else src.double())
        q, k, v = full[:, : n_q * qk], full[:, n_q * qk : (n_q + n_kv) * qk], full[:, (n_q + n_kv) * qk :]
        if norm:
            q = segedra_plain.rms_norm(q, qw.double(), 1e-5, one_plus=False)
            k = segedra_plain.rms_norm(k, kw.double(), 1e-5, one_plus=False)
        q, k = q.reshape(n, n_q, qk), k.reshape(n, n_kv, qk)
        if rot:
            q, k = (segedra_plain.rotate_pairs(t, positions, 300.0, rot) for t in (q, k))
        cache = torch.full((sum(pages_per) + 2, 2, n_kv, page_size * hd), float("nan"), dtype=dtype)
        cache_d = cache.to(DEV)
        dev = lambda t: None if t is None else t.to(DEV)  # noqa: E731
        got = ops.qk_norm_rope_write(src.to(DEV), n_q, n_kv, qk, vd, hd, dev(qw), dev(kw), 1e-5, positions.to(DEV), dev(inv_freq), dtype,
                                     cache_d, table.to(DEV), seq_of.to(DEV)).cpu()
        t = dict(rtol=3e-5, atol=3e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
        torch.testing.assert_close(got[:, :, :qk].double(), q, **t)
        assert torch.all(got[:, :, qk:] == 0)
        cache_h = cache_d.cpu()
        for row in range(n):
            pos, b = int(positions[row]), int(seq_of[row])
            k_got, v_got = cache_layout.read_kv(cache_h, int(table[b, pos // page_size]), pos % page_size, hd)
            torch.testing.assert_close(k_got[:, :qk].double(), k[row], **t)
            torch.testing.assert_close(v_got[:, :vd].double(), v[row].reshape(n_kv, vd), **t)
            assert torch.all(k_got[:, qk:] == 0) and torch.all(v_got[:, vd:] == 0)
        # queries alone (a layer that reads another's cache): the same queries, no cache touched
        alone = ops.qk_norm_rope_write(src.to(DEV), n_q, n_kv, qk, vd, hd, dev(qw), dev(kw), 1e-5, positions.to(DEV), dev(inv_freq), dtype).cpu()
        assert torch.equal(alone, got)


@pytest.mark.parametrize("experts,top", [(5, 2), (12, 12), (64, 6), (7, 1), (200, 16)])
def test_route_over_all_experts(experts, top):
    from cwm_amd import ops

    logits = rnd((300, experts), experts, 2.0)
    correction = rnd((experts,), 1, 0.2)
    s = torch.softmax(logits.double(), -1)
    for corr, renorm in ((correction, False), (None, False), (correction, True)):
        choice = s + corr.double() if corr is not None else s
        want = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
        chosen, weights = ops.route_top(logits.to(DEV), top, "softmax_all", None if corr is None else corr.to(DEV), 2.5, renorm)
        # a choice between scores closer than float32 tells apart is not tested: compare the chosen sets by their scores
        got_scores = torch.gather(choice, 1, chosen.cpu().long())
        torch.testing.assert_close(got_scores, torch.gather(choice, 1, want), rtol=1e-5, atol=1e-7)
        w = torch.gather(s, 1, chosen.cpu().long())
        if renorm:
            w = w / w.sum(-1, keepdim=True)
        torch.testing.assert_close(weights.cpu().double(), 2.5 * w, rtol=1e-5, atol=1e-8)
    # the router of the other kind is as it was
    chosen, weights = ops.route_top(logits.to(DEV), top)
    want = torch.topk(logits, top, -1)
    assert torch.equal(chosen.cpu().long(), want.indices)
    torch.testing.assert_close(weights.cpu(), torch.softmax(want.values, -1), rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tokens,experts,top,dim,ff", [(5, 6, 2, 40, 24), (300, 3, 2, 64, 48), (1500, 2, 2, 128, 100), (700, 4, 1, 48, 20)])
def test_clamped_gated_product(dtype, tokens, experts, top, dim, ff):
    """The three shapes of the grouped product (few rows an expert, 64 and more, 256 and more with K a multiple of 64)."""
    from cwm_amd import ops

    x = rnd((tokens, dim), 1).to(dtype)
    gate, up = rnd((experts, ff, dim), 2, 0.3).to(dtype), rnd((experts, ff, dim), 3, 0.3).to(dtype)
    g = torch.Generator().manual_seed(4)
    chosen = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(tokens)]).to(torch.int32)
    groups = ops.group_by_expert(chosen.to(DEV), experts)
    act = ops.GatedActivation("clamped_swish", 1.702, 0.8)
    rows = ops.grouped_gate_up(x.to(DEV), groups, gate.to(DEV), up.to(DEV), act).cpu()
    pair_row = groups.pair_row.cpu().long().view(tokens, top)
    e = chosen.long()
    gg = torch.einsum("td,tkfd->tkf", x.double(), gate.double()[e]).clamp(max=0.8)
    uu = torch.einsum("td,tkfd->tkf", x.double(), up.double()[e]).clamp(-0.8, 0.8)
    want = gg * torch.sigmoid(1.702 * gg) * (uu + 1)
    assert (gg == 0.8).any() and (uu.abs() == 0.8).any()  # the limits are reached
    torch.testing.assert_close(rows[pair_row].double(), want, **(dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)))
    # and silu(g) * u where no activation is named, as before
    rows = ops.grouped_gate_up(x.to(DEV), groups, gate.to(DEV), up.to(DEV)).cpu()
    gg = torch.einsum("td,tkfd->tkf", x.double(), gate.double()[e])
    want = gg * torch.sigmoid(gg) * torch.einsum("td,tkfd->tkf", x.double(), up.double()[e])
    torch.testing.assert_close(rows[pair_row].double(), want, **(dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)))


def _sink_case(dtype, n_q, n_kv, hd, page_size, lens_old, lens_new, window, seed, loud=None):
    """Keys, values and queries of a mixed batch in a shuffled paged cache, and float64 attention with a sink on the device."""
    g = torch.Generator().manual_seed(seed)
    scale = hd ** -0.5
    sink = torch.rand(n_q, generator=g) * 9.0 - 1.0
    pages_per = [(a + b + page_size - 1) // page_size for a, b in zip(lens_old, lens_new)]
    total = sum(pages_per) + 1
    perm = torch.randperm(total, generator=g)
    table = torch.full((len(lens_old), max(pages_per)), -1, dtype=torch.int32)
    cache = torch.full((total, 2, n_kv, page_size * hd), float("nan"), dtype=dtype)
    vb = 8 if page_size % 8 == 0 else page_size
    kc = cache[:, 0].view(total, n_kv, page_size, hd)
    vc = cache[:, 1].view(total, n_kv, page_size // vb, hd, vb)
    used, q_rows, want_rows = 0, [], []
    group = n_q // n_kv
    for b, (n0, n1) in enumerate(zip(lens_old, lens_new)):
        n = n0 + n1
        k = torch.randn((n, n_kv, hd), generator=g).to(dtype)
        v = torch.randn((n, n_kv, hd), generator=g).to(dtype)
        q = torch.randn((n1, n_q, hd), generator=g).to(dtype)
        for lb, key_pos in ([loud] if isinstance(loud, tuple) else (loud or [])):
            if lb == b:  # a key that answers the last query's first heads loudly (those of key/value head 0)
                k[key_pos, 0] = (q[-1, 0].float() * 6.0).to(dtype)
        table[b, : pages_per[b]] = perm[used : used + pages_per[b]].to(torch.int32)
        used += pages_per[b]
        pos = torch.arange(n)
        pages, slots = table[b, pos // page_size].long(), pos % page_size
        kc[pages, :, slots, :] = k
        vc[pages, :, slots // vb, :, slots % vb] = v
        kd, vd, qd = k.double().to(DEV), v.double().to(DEV), q.double().to(DEV)
        scores = torch.einsum("thd,khd->htk", qd, kd.repeat_interleave(group, dim=1)) * scale
        qpos = torch.arange(n0, n, device=DEV).view(1, -1, 1)
        kpos = torch.arange(n, device=DEV).view(1, 1, -1)
        ok = kpos <= qpos
        if window is not None:
            ok = ok & (kpos >= qpos - (window - 1))
        scores = scores.masked_fill(~ok, float("-inf"))
        with_sink = torch.cat([scores, sink.double().to(DEV).view(n_q, 1, 1).expand(n_q, n1, 1)], -1)
        probs = torch.softmax(with_sink, -1)[..., :-1]
        want_rows.append(torch.einsum("htk,khd->thd", probs, vd.repeat_interleave(group, dim=1)).reshape(n1, -1).cpu())
        q_rows.append(q)
    kv_lens = [a + b for a, b in zip(lens_old, lens_new)]
    cu = [0]
    for n in lens_new:
        cu.append(cu[-1] + n)
    batch = SimpleNamespace(
        q_lens=lens_new, kv_lens=kv_lens, n_seqs=len(kv_lens), n_tokens=sum(lens_new), scratch={}, max_kv_len=max(kv_lens),
        cu_q=torch.tensor(cu, dtype=torch.int32).to(DEV), kv_len=torch.tensor(kv_lens, dtype=torch.int32).to(DEV),
        positions=torch.cat([torch.arange(a, a + b) for a, b in zip(lens_old, lens_new)]).to(torch.int32).to(DEV),
        seq_of_token=torch.cat([torch.full((n,), b) for b, n in enumerate(lens_new)]).to(torch.int32).to(DEV),
    )
    return torch.cat(q_rows).to(DEV), cache.to(DEV), table.to(DEV), batch, sink.to(DEV), scale, torch.cat(want_rows)


@pytest.mark.parametrize("window", [None, 9, 300])
@pytest.mark.parametrize("n_q,n_kv,hd,page_size", [(4, 2, 16, 8), (3, 1, 32, 16), (12, 2, 128, 64), (6, 3, 80, 16), (8, 8, 64, 32), (5, 5, 48, 5)])
def test_attention_sink_in_both_kernels(n_q, n_kv, hd, page_size, window):
    """A fresh prompt, continued portions, decoded tokens near and far into their sequences and a long portion: every
    row's softmax holds its head's sink once, in the matrix-core kernels and in the plain kernel in both types."""
    from cwm_amd import ops

    lens_old, lens_new = [0, 37, 70, 700, 520, 13], [29, 21, 1, 1, 3, 200]
    for dtype in DTYPES:
        q, cache, table, batch, sink, scale, want = _sink_case(dtype, n_q, n_kv, hd, page_size, lens_old, lens_new, window, seed=hd + n_q)
        t = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
        simple = ops.paged_attention_simple(q, cache, table, batch.positions, batch.seq_of_token, window, scale, sink=sink).cpu()
        torch.testing.assert_close(simple.double(), want, **t)
        without = ops.paged_attention_simple(q, cache, table, batch.positions, batch.seq_of_token, window, scale).cpu()
        assert (without.double() - want).abs().max() > 0.05  # the sink matters in this case
        if dtype == torch.bfloat16 and ops.mfma_attention_takes(dtype, hd, page_size):
            got = ops.paged_attention_mfma(q, cache, table, batch, window, scale, sink).cpu()
            assert torch.isfinite(got).all()
            torch.testing.assert_close(got.double(), want, **t)
            torch.testing.assert_close(got.float(), simple.float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("window", [None, 5000])
def test_attention_sink_where_key_ranges_are_cut_and_merged(window):
    """Decoded tokens and portions far into long sequences: the matrix-core kernel cuts their keys into chunks and a
    second kernel merges the partial results, the plain kernel cuts into segments: the sink counts once all the same.
    One far key stands out against the sink."""
    from cwm_amd import ops

    n_q, n_kv, hd, page_size = 6, 2, 64, 64
    lens_old, lens_new = [9000, 3000, 1500, 20000, 6000], [1, 2, 1, 150, 1400]
    q, cache, table, batch, sink, scale, want = _sink_case(torch.bfloat16, n_q, n_kv, hd, page_size, lens_old, lens_new, window, seed=5, loud=(0, 4321))
    got = ops.paged_attention_mfma(q, cache, table, batch, window, scale, sink).cpu()
    assert torch.isfinite(got).all()
    torch.testing.assert_close(got.double(), want, rtol=2e-2, atol=2e-2)
    simple = ops.paged_attention_simple(q, cache, table, batch.positions, batch.seq_of_token, window, scale, sink=sink).cpu()
    torch.testing.assert_close(simple.double(), want, rtol=2e-2, atol=2e-2)
    without = ops.paged_attention_mfma(q, cache, table, batch, window, scale).cpu()
    assert (without.double() - want).abs().max() > 0.02


@pytest.mark.parametrize("window,page_size", [(64, 16), (40, 8), (33, 32), (2, 16)])
def test_attention_sink_and_a_loud_key_at_the_window_s_edges(window, page_size):
    """The last query of a decoded token and of a prompt portion finds a loud key exactly at the window's first place
    (it carries the row, sink or not) or one place before it (it must not be seen): a window one key off in either
    direction changes these rows altogether.  With a window of 64 the edge lies at a page border."""
    from cwm_amd import ops

    n_q, n_kv, hd = 4, 2, 64
    lens_old, lens_new = [300, 300, 171, 171], [1, 1, 37, 37]
    last = [a + b - 1 for a, b in zip(lens_old, lens_new)]
    loud = [(0, last[0] - (window - 1)), (1, last[1] - window), (2, last[2] - (window - 1)), (3, last[3] - window)]
    for dtype in DTYPES:
        q, cache, table, batch, sink, scale, want = _sink_case(dtype, n_q, n_kv, hd, page_size, lens_old, lens_new, window, seed=window, loud=loud)
        # the case is sharp: had the query of sequence 1 (or 3) seen the key one place before its window, its row would be another
        longer = _sink_case(dtype, n_q, n_kv, hd, page_size, lens_old, lens_new, window + 1, seed=window, loud=loud)[-1]
        shorter = _sink_case(dtype, n_q, n_kv, hd, page_size, lens_old, lens_new, window - 1, seed=window, loud=loud)[-1] if window > 1 else None
        rows = {0: 0, 1: 1, 2: 2 + 36, 3: 2 + 37 + 36}  # the last row of each sequence
        assert (longer[rows[1]] - want[rows[1]]).abs().max() > 0.3 and (longer[rows[3]] - want[rows[3]]).abs().max() > 0.3
        if shorter is not None:
            assert (shorter[rows[0]] - want[rows[0]]).abs().max() > 0.3 and (shorter[rows[2]] - want[rows[2]]).abs().max() > 0.3
        t = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
        simple = ops.paged_attention_simple(q, cache, table, batch.positions, batch.seq_of_token, window, scale, sink=sink).cpu()
        torch.testing.assert_close(simple.double(), want, **t)
        if dtype == torch.bfloat16:
            got = ops.paged_attention_mfma(q, cache, table, batch, window, scale, sink).cpu()
            torch.testing.assert_close(got.double(), want, **t)


# ---- models ------------------------------------------------------------------------------------------------------- #
LENGTHS = {"tiny_s": [1, 6, 21, 70, 130], "tiny_t": [9, 33, 2, 100, 57], "tiny_u": [150, 41, 90]}
PAGE_SIZES = {"whole": 16, "tail": 16, "portions": 8, "mixed": 8}


def requests_for(name, lengths=None):
    vocab = segedra.get(name)["vocab"]
    return {f"r{i}": traces.random_tokens(13 * i + len(name), n, vocab) for i, n in enumerate(lengths or LENGTHS[name])}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("segedra")
    return {name: segedra.make_folder(root, name, seed=5) for name in segedra.ALL}


@pytest.fixture(scope="module")
def plain_cache():
    return {}


def plain_for(folders, cache, name, dtype):
    if (name, dtype) not in cache:
        cache[name, dtype] = segedra.expected(folders[name], requests_for(name), dtype)
    return cache[name, dtype]


def run(folder, dtype, steps, requests, vocab, **options):
    from cwm_amd.replay import Replayer

    rep = Replayer(folder, dtype, traces.max_live_tokens(steps), poison_freed_pages=True, **options)
    page_use = traces.PageUse(rep.manager)
    outputs = traces.run_in_process(rep, steps, page_use)
    assert rep.manager.live_requests() == []
    return traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab), rep, page_use


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(segedra.ALL))
@pytest.mark.parametrize("regime", ["whole", "tail", "portions", "mixed"])
def test_replay_regimes(folders, plain_cache, name, dtype, regime):
    requests = requests_for(name)
    vocab = segedra.get(name)["vocab"]
    steps = {"whole": traces.whole, "tail": traces.tail_one_by_one, "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, max_live=3)}[regime](requests)
    got, rep, page_use = run(folders[name], dtype, steps, requests, vocab, page_size=PAGE_SIZES[regime], max_requests=3 if regime == "mixed" else 16)
    want = plain_for(folders, plain_cache, name, dtype)
    for rid in requests:
        segedra.check(got[rid], want[rid], dtype, f"{name} {dtype} {regime} {rid}")
    if regime == "mixed":
        for g in rep.manager.groups:
            assert page_use.pages_shared_between_requests(g.index) > 0, f"group {g.index}: no page served two requests"


def single_layer(layer: dict, width: int = 40, vocab: int = 83, streams=2, loop=None) -> dict:
    config = {"architecture": "Segedra", "vocab": vocab, "width": width, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0}, "layers": [layer]}
    if streams is not None:
        config["streams"] = streams
    if loop is not None:
        config["loop"] = loop
    return config


SINGLE_LAYERS = {
    "attention_alone": single_layer(segedra.attn(4, 2, 8, 8, 0.5, window=6, rot=(100.0, 8))),
    "attention_unequal_heads_partly_rotated": single_layer(segedra.attn(3, 1, 20, 36, 0.4, window=25, rot=(3000.0, 6)), streams=None),
    "attention_window_of_a_page": single_layer(segedra.attn(2, 2, 16, 16, 1.5, window=8, rot=(10.0, 16)), streams=1),
    "attention_heads_of_a_hundred_and_twelve": single_layer(segedra.attn(2, 1, 112, 100, 0.1, window=40, rot=(500.0, 112)), streams=2),
    "attention_sizes_that_are_no_multiple_of_four": single_layer(segedra.attn(3, 3, 10, 6, 0.4, window=9, rot=(70.0, 6), mlp=segedra.dense(21)), width=50, vocab=67, streams=3),
    "dense": single_layer(segedra.attn(1, 1, 4, 4, 0.5, window=2, rot=(10.0, 2), mlp=segedra.dense(72)), streams=4),
    "experts_all": single_layer(segedra.attn(1, 1, 4, 4, 0.5, window=2, rot=(10.0, 2), mlp=segedra.moe(12, 4, 4, 0.6, 0.5)), streams=3),
    "experts_one_of_many": single_layer(segedra.attn(1, 1, 4, 4, 0.5, window=2, rot=(10.0, 2), mlp=segedra.moe(30, 20, 1, 3.0, 4.0)), streams=None),
    "one_layer_five_times": single_layer(segedra.attn(2, 2, 8, 12, 0.6, window=5, rot=(50.0, 4), mlp=segedra.dense(24)), streams=2,
                                          loop={"start": 0, "stop": 1, "times": 5}),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", list(SINGLE_LAYERS))
def test_single_layers(tmp_path, which, dtype):
    """One mechanism at a time between embedding and head: whole prompts against the same tokens in portions and one
    by one, and both against the plain implementation."""
    config = SINGLE_LAYERS[which]
    folder = segedra.make_folder(tmp_path, which, seed=2, config=config)
    requests = {f"r{i}": traces.random_tokens(i + 5, n, config["vocab"]) for i, n in enumerate([37, 5, 64])}
    want = segedra.expected(folder, requests, dtype)
    for make in (traces.whole, traces.portions, lambda r: traces.tail_one_by_one(r, tail=20)):
        steps = make(requests)
        got, _, _ = run(folder, dtype, steps, requests, config["vocab"], page_size=8)
        for rid in requests:
            segedra.check(got[rid], want[rid], dtype, f"{which} {dtype} {rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_over_long_sequences(folders, dtype):
    """tiny_t's softmax is sharp: a token's result hangs on single keys, hundreds of places back in the layer that
    reads every key, and at the windows' first and last keys in the others (a window one key too long or too short
    takes in or loses such a key).  A prompt of 700 tokens whole, in portions that end at, before and after page
    borders, and with its last 150 tokens one by one."""
    name = "tiny_t"
    vocab = segedra.get(name)["vocab"]
    requests = {"long": traces.random_tokens(99, 700, vocab)}
    want = segedra.expected(folders[name], requests, dtype)
    portions = lambda r: traces.portions(r, sizes=[64, 63, 65, 2, 126, 1, 31, 33, 128, 17])  # noqa: E731
    for make in (traces.whole, portions, lambda r: traces.tail_one_by_one(r, tail=150)):
        steps = make(requests)
        got, _, _ = run(folders[name], dtype, steps, requests, vocab, page_size=32)
        segedra.check(got["long"], want["long"], dtype, f"{name} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_wider_layers_and_many_rows(tmp_path, dtype):
    """Width 256 and prompts of 600 and 300 tokens: the kernels' shapes for many rows, whole, in large portions beside
    each other, and with a tail of single tokens."""
    config = segedra.MEDIUM
    folder = segedra.make_folder(tmp_path, "medium", seed=9, config=config)
    vocab = config["vocab"]
    requests = {"a": traces.random_tokens(31, 600, vocab), "b": traces.random_tokens(32, 300, vocab)}
    want = segedra.expected(folder, requests, dtype)
    side_by_side = [
        {"step": 0, "entries": [{"id": "a", "tokens": requests["a"][:290], "want": list(range(290))}, {"id": "b", "tokens": requests["b"][:270], "want": list(range(270))}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": requests["a"][290:], "want": list(range(310))}, {"id": "b", "tokens": requests["b"][270:], "want": list(range(30))}], "end": ["a", "b"]},
    ]
    for steps in (traces.whole(requests), side_by_side, traces.tail_one_by_one(requests, tail=20)):
        got, _, _ = run(folder, dtype, steps, requests, vocab, page_size=32)
        for rid in requests:
            segedra.check(got[rid], want[rid], dtype, f"medium {dtype} {rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decoding(folders, dtype):
    """Every token a step of its own from an empty cache, for 300 steps: the windows pass over decoded tokens and
    give their pages back on the way."""
    name = "tiny_s"
    vocab = segedra.get(name)["vocab"]
    requests = {"a": traces.random_tokens(4, 300, vocab)}
    steps = traces.tail_one_by_one(requests, tail=299)
    got, _, _ = run(folders[name], dtype, steps, requests, vocab, page_size=16)
    segedra.check(got["a"], segedra.expected(folders[name], requests, dtype)["a"], dtype, f"{name} {dtype} one by one")


def test_pages_that_are_used_again_hold_nothing_of_their_first_user(folders):
    """A pool of the second request's size only: it takes the pages the first one gave back, NaN in between."""
    name = "tiny_u"
    vocab = segedra.get(name)["vocab"]
    a, b = traces.random_tokens(1, 60, vocab), traces.random_tokens(2, 25, vocab)
    both = [
        {"step": 0, "entries": [{"id": "a", "tokens": a, "want": [59]}], "end": ["a"]},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:10], "want": list(range(10))}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[10:], "want": list(range(15))}], "end": ["b"]},
    ]
    got, rep, _ = run(folders[name], "float32", both, {"a": a, "b": b}, vocab, page_size=8, max_requests=1)
    alone, _, _ = run(folders[name], "float32", both[1:], {"b": b}, vocab, page_size=8, max_requests=1)
    assert np.array_equal(got["b"], alone["b"])
    segedra.check(got["b"], segedra.expected(folders[name], {"b": b}, "float32")["b"], "float32", "second user of the pages")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_logits_do_not_depend_on_the_rest_of_the_batch(folders, dtype):
    """A request's decoded tokens alone and beside two other requests' portions: the same bits."""
    name = "tiny_s"
    vocab = segedra.get(name)["vocab"]
    r = requests_for(name, [40, 64, 90])
    alone = [{"step": 0, "entries": [{"id": "r0", "tokens": r["r0"][:30], "want": [29]}], "end": []}] + [
        {"step": 1 + i, "entries": [{"id": "r0", "tokens": [r["r0"][30 + i]], "want": [0]}], "end": ["r0"] if i == 9 else []} for i in range(10)
    ]
    beside = [{"step": 0, "entries": [{"id": "r0", "tokens": r["r0"][:30], "want": [29]}], "end": []}]
    for i in range(10):
        entries = [{"id": "r1", "tokens": r["r1"][6 * i : 6 * i + 6], "want": [5]}, {"id": "r0", "tokens": [r["r0"][30 + i]], "want": [0]},
                   {"id": "r2", "tokens": r["r2"][9 * i : 9 * i + 9], "want": []}]
        beside.append({"step": 1 + i, "entries": entries, "end": ["r0", "r1", "r2"] if i == 9 else []})
    lengths = {"r0": r["r0"][:40], "r1": r["r1"][:60], "r2": r["r2"][:90]}
    got_alone, _, _ = run(folders[name], dtype, alone, {"r0": lengths["r0"]}, vocab, page_size=8)
    got_beside, _, _ = run(folders[name], dtype, beside, lengths, vocab, page_size=8)
    assert np.array_equal(got_alone["r0"][29:], got_beside["r0"][29:])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_replayed_from_graphs_give_the_same_bits(folders, dtype):
    name = "tiny_s"
    vocab = segedra.get(name)["vocab"]
    requests = requests_for(name, [30, 44, 37])
    heads = {"step": 0, "entries": [{"id": r, "tokens": t[:20], "want": [19]} for r, t in requests.items()], "end": []}
    steps = [heads] + [
        {"step": 1 + i, "entries": [{"id": r, "tokens": [t[20 + i]], "want": [0]} for r, t in requests.items()], "end": list(requests) if i == 9 else []}
        for i in range(10)
    ]
    launched, _, _ = run(folders[name], dtype, steps, {k: v[:30] for k, v in requests.items()}, vocab, page_size=16)
    replayed, rep, _ = run(folders[name], dtype, steps, {k: v[:30] for k, v in requests.items()}, vocab, page_size=16, num_graphs=2)
    assert rep.runner.n_replays >= 8, "the decode steps were not replayed"
    for rid in requests:
        assert np.array_equal(launched[rid][19:], replayed[rid][19:]), rid


def plain_greedy(folder, prompt, n_new):
    config, weights = segedra.read_folder(folder)
    toks, out = list(prompt), []
    for _ in range(n_new):
        logits = segedra_plain.forward(weights, config, toks, torch.float64)[-1]
        out.append(int(torch.argmax(logits)))
        toks.append(out[-1])
    return out


@pytest.mark.parametrize("name", ["tiny_s", "tiny_u"])
def test_greedy_generation_through_the_engine(folders, name):
    """The engine's own entry point: scheduler, portions of 24 tokens, continuous batching, sampling kernel; then a
    cache that holds barely more than the longest request, so that requests wait for one another's pages."""
    from cwm_amd.engine import Engine, GenArgs

    vocab = segedra.get(name)["vocab"]
    prompts = [traces.random_tokens(20 + i, n, vocab) for i, n in enumerate([5, 17, 33, 64])]
    engine = Engine.from_folder(folders[name], GenArgs(use_sampling=False, max_batch=4, max_seq=2048, cache_block=16, max_prefill=24), dtype="float32")
    got = engine.generate_tokens(prompts, max_gen=12)
    for p, g in zip(prompts, got):
        assert g == plain_greedy(folders[name], p, 12)
    small = Engine.from_folder(folders[name], GenArgs(use_sampling=False, max_batch=4, max_seq=96, cache_block=4, max_prefill=24), dtype="float32")
    assert small.generate_tokens(prompts, max_gen=12) == got


def test_command_line_and_trace_run_as_child_processes(folders, tmp_path):
    name = "tiny_s"
    vocab = segedra.get(name)["vocab"]
    prompts = [traces.random_tokens(60 + i, n, vocab) for i, n in enumerate([6, 21])]
    path = tmp_path / "prompts.jsonl"
    path.write_text("".join(json.dumps({"id": i, "tokens": p}) + "\n" for i, p in enumerate(prompts)))
    cmd = [sys.executable, "-m", "cwm_amd.generate", f"checkpoint_dir={folders[name]}", f"prompts={path}", "dtype=float32",
           "gen_args.use_sampling=false", "gen_args.max_gen=7", "gen_args.max_seq=512", "gen_args.cache_block=16", "gen_args.max_batch=4"]
    res = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr
    got = {rec["id"]: rec["tokens"] for rec in map(json.loads, res.stdout.strip().splitlines())}
    for i, p in enumerate(prompts):
        assert got[i] == plain_greedy(folders[name], p, 7)

    requests = requests_for(name, [40, 75, 33])
    steps = traces.mixed(requests)
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / f"out_{dtype}"
        cmd = [os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name], "--dtype", dtype, "--out", str(out),
               "--max-tokens", str(traces.max_live_tokens(steps))]
        res = subprocess.run(cmd, input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
        assert res.returncode == 0, res.stderr
        assert [line for line in res.stdout.splitlines() if line.startswith("done")] == [f"done {s['step']}" for s in steps]
        outputs = {s["step"]: np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(-1, vocab) for s in steps if any(e["want"] for e in s["entries"])}
        got = traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab)
        want = segedra.expected(folders[name], requests, dtype)
        for rid in requests:
            segedra.check(got[rid], want[rid], dtype, f"trace_run {dtype} {rid}")


def random_config(seed: int) -> dict:
    """A configuration drawn from a seed: every size, count, constant and the order of layers differ from draw to draw."""
    import random

    rng = random.Random(seed)
    width = rng.choice([32, 40, 48, 64, 72, 96, 100, 128, 136, 192, 200, 256])
    layers = []
    for _ in range(rng.randint(2, 5)):
        kv = rng.choice([1, 2, 3, 4])
        heads = kv * rng.choice([1, 2, 3, 4])
        dim = rng.choice([8, 16, 24, 32, 40, 48, 64, 72, 96, 128])
        vdim = rng.choice([8, 12, 16, 32, 48, 64, 80, 128])
        rot = (rng.choice([100.0, 10000.0, 250000.0, 1e6]), rng.choice([d for d in (2, 4, 8, 16, 32, 64, 128) if d <= dim] + [dim]))
        kind = rng.choice(["dense", "moe", "moe", "none"])
        if kind == "dense":
            mlp = segedra.dense(rng.choice([20, 36, 64, 100, 256]))
        elif kind == "moe":
            experts = rng.randint(2, 12)
            mlp = segedra.moe(rng.choice([8, 12, 32, 50, 64]), experts, rng.randint(1, experts), rng.choice([0.5, 1.0, 2.0, 7.0]), rng.choice([0.5, 1.0, 2.5]))
        else:
            mlp = None
        window = rng.choice([None, 1, 2, 7, 16, 17, 40, 64, 100])
        layers.append(segedra.attn(heads, kv, dim, vdim, rng.choice([0.05, 0.1, 0.2]) * (64 / dim) ** 0.5, window=window, rot=rot, mlp=mlp))
    config = {"architecture": "Segedra", "vocab": rng.randint(50, 700), "width": width, "norm": {"eps": rng.choice([1e-5, 1e-6])},
              "embedding": {"scale": rng.choice([0.7, 1.0, 1.5]) * width ** 0.5}, "layers": layers}
    if rng.random() < 0.8:
        config["streams"] = rng.randint(1, 5)
    if rng.random() < 0.7:
        start = rng.randint(0, len(layers) - 1)
        config["loop"] = {"start": start, "stop": rng.randint(start + 1, len(layers)), "times": rng.randint(1, 3)}
    return config


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(10))
def test_random_configurations(tmp_path, seed, dtype):
    """Other models of the design: whole prompts, and a mixed schedule with pages of another size, against the plain
    implementation."""
    config = random_config(seed)
    folder = segedra.make_folder(tmp_path, f"random{seed}", seed=seed, config=config)
    vocab = config["vocab"]
    requests = {f"r{i}": traces.random_tokens(7 * seed + i, n, vocab) for i, n in enumerate([3, 150, 45, 88])}
    want = segedra.expected(folder, requests, dtype)
    for steps, page in ((traces.whole(requests), 16), (traces.mixed(requests, max_live=3), 32 if seed % 2 else 8)):
        got, _, _ = run(folder, dtype, steps, requests, vocab, page_size=page, max_requests=4)
        for rid in requests:
            segedra.check(got[rid], want[rid], dtype, f"random configuration {seed} {dtype} {rid}: {json.dumps(config)}")
