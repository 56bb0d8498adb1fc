"""Each kernel of the layers with group norms, token shift, a selective state space and routed experts, alone,
against a plain float32 PyTorch computation of the same operation (`tests/helpers/cpu_ops.py`)."""

from types import SimpleNamespace

import pytest
import torch

from helpers import cpu_ops

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = {torch.float32: dict(rtol=2e-5, atol=2e-5), torch.bfloat16: dict(rtol=2e-2, atol=2e-2)}


def _batch(q_lens, starts, slots, device):
    """A step's vectors for sequences that bring `q_lens` tokens after `starts` cached ones."""
    cu = [0]
    for q in q_lens:
        cu.append(cu[-1] + q)
    seq = [b for b, q in enumerate(q_lens) for _ in range(q)]
    pos = [s + i for s, q in zip(starts, q_lens) for i in range(q)]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)  # noqa: E731
    return SimpleNamespace(n_tokens=cu[-1], n_seqs=len(q_lens), cu_q=i32(cu), seq_of_token=i32(seq), positions=i32(pos), state_slots=i32(slots),
                           q_lens=list(q_lens), scratch={})


def _both(q_lens, starts, slots):
    return _batch(q_lens, starts, slots, DEV), _batch(q_lens, starts, slots, "cpu")


def _close(got, want, dtype, what):
    torch.testing.assert_close(got.float().cpu(), want.float(), msg=lambda m: f"{what}: {m}", **TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dim,groups", [(160, 4), (96, 1), (1000, 5), (4096, 2), (24, 24)])
def test_group_norm_forms(dtype, dim, groups):
    from cwm_amd import ops

    torch.manual_seed(dim + groups)
    x = torch.randn(7, dim) * 3
    w = torch.rand(dim) + 0.5
    xd, wd = x.to(DEV, dtype), w.to(DEV, dtype)
    xr, wr = xd.cpu(), wd.cpu()
    _close(ops.group_rmsnorm(xd, wd, groups, 1e-5, dtype), cpu_ops.group_rmsnorm(xr, wr, groups, 1e-5, torch.float32), dtype, "fresh")
    rows = torch.tensor([5, 0, 3], dtype=torch.int32)
    _close(ops.group_rmsnorm(xd, wd, groups, 1e-5, dtype, rows=rows.to(DEV)), cpu_ops.group_rmsnorm(xr, wr, groups, 1e-5, torch.float32, rows=rows), dtype, "rows")
    # partial sums added in order, into the float32 stream
    parts = torch.randn(3, 7, dim)
    h = torch.randn(7, dim)
    hd = h.to(DEV)
    also = torch.empty(7, dim, dtype=dtype, device=DEV)
    ops.group_rmsnorm(parts.to(DEV), wd, groups, 1e-5, torch.float32, out=hd, accumulate=True, copy=also)
    want = cpu_ops.group_rmsnorm(parts, wr, groups, 1e-5, torch.float32, out=h.clone(), accumulate=True)
    _close(hd, want, torch.float32, "accumulate")
    assert torch.equal(also, hd.to(dtype))  # the stream as it now stands, in the activation type
    # in place on columns of a wider tensor; the other columns stay
    wide = (torch.randn(7, dim + 40) * 2).to(DEV, dtype)
    keep = wide.clone()
    ops.group_rmsnorm(wide[:, 24 : 24 + dim], wd, groups, 1e-5, dtype, out=wide[:, 24 : 24 + dim])
    _close(wide[:, 24 : 24 + dim], cpu_ops.group_rmsnorm(keep[:, 24 : 24 + dim].cpu(), wr, groups, 1e-5, torch.float32), dtype, "in place")
    assert torch.equal(wide[:, :24], keep[:, :24]) and torch.equal(wide[:, 24 + dim :], keep[:, 24 + dim :])
    # the gate comes before the norm
    gate = torch.randn(7, dim).to(DEV, dtype)
    y = torch.randn(7, dim).to(DEV)
    _close(ops.group_rmsnorm(y, wd, groups, 1e-5, dtype, gate=gate), cpu_ops.group_rmsnorm(y.cpu(), wr, groups, 1e-5, torch.float32, gate=gate.cpu()), dtype, "gated")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_shift_first_tokens_and_state(dtype):
    from cwm_amd import ops

    torch.manual_seed(3)
    dim = 200
    q_lens, starts, slots = [1, 5, 2, 1], [0, 0, 9, 4], [3, 0, 2, 1]
    gb, cb = _both(q_lens, starts, slots)
    h = torch.randn(sum(q_lens), dim)
    mu = torch.rand(dim)
    state = torch.randn(4, dim)
    sd = state.to(DEV)
    got = ops.token_shift(h.to(DEV), mu.to(DEV), sd, gb, dtype)
    want = cpu_ops.token_shift(h, mu, state, cb, torch.float32)
    _close(got, want, dtype, "shift")
    _close(sd, state, torch.float32, "state")
    # position 0 ignores whatever the slot held; later portions start from it
    assert torch.allclose(want[0], h[0] * (1 - mu))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
@pytest.mark.parametrize("channels", [300, 320])
def test_causal_conv_against_whole_sequence(dtype, taps, channels):
    """Portions of 1, 2, 3 and more tokens carry the convolution's inputs through the state (320 channels in rows of a
    multiple of 16 bytes: the path that fetches eight channels at once)."""
    from cwm_amd import ops

    torch.manual_seed(taps)
    offset, n = 17, 23
    x = torch.randn(n, channels).to(dtype)
    w, b = torch.randn(channels, taps), torch.randn(channels)
    whole_state = torch.zeros(2, offset + (taps - 1) * channels + 5)
    whole = cpu_ops.causal_conv_silu(x.float(), w, b, whole_state, offset, _batch([n], [0], [1], "cpu"))
    state = torch.zeros_like(whole_state).to(DEV)
    state[0] = 7.0  # another request's slot
    at, outs = 0, []
    for q in (1, 2, 1, 3, 9, 2, 5):
        lead = 3 if channels % 8 else 8
        wide = torch.randn(q, channels + 16).to(DEV, dtype)  # rows that lie apart
        wide[:, lead : lead + channels] = x[at : at + q].to(DEV)
        outs.append(ops.causal_conv_silu(wide[:, lead : lead + channels], w.to(DEV), b.to(DEV), state, offset, _batch([q], [at], [1], DEV), w.t().contiguous().to(DEV)))
        at += q
    _close(torch.cat(outs), whole, dtype, "portions")
    _close(state[1], whole_state[1], torch.float32, "state")
    assert torch.all(state[0] == 7.0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,head_dim,n_state,groups", [(4, 40, 56, 2), (3, 20, 5, 1), (2, 64, 128, 2), (6, 8, 200, 3), (1, 130, 16, 1)])
def test_selective_scan_batch_and_portions(dtype, heads, head_dim, n_state, groups):
    from cwm_amd import ops

    torch.manual_seed(heads * 7 + n_state)
    inner, width = heads * head_dim, heads * head_dim + 2 * groups * n_state  # noqa: F841
    q_lens, starts, slots = [5, 1, 12], [0, 3, 40], [2, 0, 1]
    n = sum(q_lens)
    xbc = torch.randn(n, width).to(dtype)
    dt = (torch.randn(n, heads) - 1).to(dtype)
    dt_bias, a_log, d_skip = torch.randn(heads) * 0.5, torch.randn(heads) * 0.5, torch.randn(heads)
    elems = heads * n_state * head_dim
    state = torch.randn(3, elems + 11)
    state[2, :elems] = 0  # the sequence that starts
    # the kernel keeps a head's state in an order and padding of its own
    n_dev = -(-(ops.scan_state_elems(heads, head_dim, n_state) + 11) // 4) * 4
    pack = lambda rows: torch.stack([ops.scan_state_pack(r[:elems].reshape(heads, n_state, head_dim)) for r in rows])  # noqa: E731
    sd = torch.full((3, n_dev), 5.0)
    sd[:, : ops.scan_state_elems(heads, head_dim, n_state)] = pack(state)
    sd = sd.to(DEV)
    gb, cb = _both(q_lens, starts, slots)
    wide = torch.zeros(n, width + heads + 6, dtype=dtype, device=DEV)
    wide[:, :width], wide[:, width : width + heads] = xbc.to(DEV), dt.to(DEV)
    args = (dt_bias.to(DEV), a_log.to(DEV), d_skip.to(DEV))
    got = ops.selective_scan(wide[:, :width], wide[:, width : width + heads], *args, sd, gb, heads, head_dim, n_state, groups)
    want = cpu_ops.selective_scan(xbc.float(), dt.float(), dt_bias, a_log, d_skip, state, cb, heads, head_dim, n_state, groups)
    tol = dict(rtol=2e-4, atol=2e-4)
    torch.testing.assert_close(got.cpu(), want, **tol)
    for slot in range(3):
        torch.testing.assert_close(ops.scan_state_unpack(sd[slot].cpu(), heads, head_dim, n_state).reshape(-1), state[slot, :elems], **tol)
    assert torch.all(sd[:, ops.scan_state_elems(heads, head_dim, n_state) :] == 5.0)  # what lies behind the heads' states is not touched
    # the same tokens one by one give the same bits as the portion did (the first sequence again, from zero)
    sd2 = torch.zeros((3, n_dev), device=DEV)
    singles = []
    for i in range(5):
        one = _batch([1], [i], [2], DEV)
        singles.append(ops.selective_scan(wide[i : i + 1, :width], wide[i : i + 1, width : width + heads], *args, sd2, one, heads, head_dim, n_state, groups))
    assert torch.equal(torch.cat(singles), got[:5])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,head_dim,n_state,groups", [(2, 16, 24, 1), (2, 64, 128, 2)])
def test_selective_scan_long_portions_in_segments(dtype, heads, head_dim, n_state, groups):
    """Portions longer than a segment run their segments side by side: a long fresh prompt, a decoded token and a
    long portion that goes on from a state, in one step; the end states carry on into a second step."""
    from cwm_amd import ops

    torch.manual_seed(n_state)
    inner, width = heads * head_dim, heads * head_dim + 2 * groups * n_state  # noqa: F841
    elems, dev_elems = heads * n_state * head_dim, ops.scan_state_elems(heads, head_dim, n_state)
    dt_bias, a_log, d_skip = torch.randn(heads) * 0.5 - 1, torch.rand(heads) * -3 - 1, torch.randn(heads)
    args = (dt_bias.to(DEV), a_log.to(DEV), d_skip.to(DEV))
    state = torch.randn(3, elems) * 0.3
    state[0] = 0
    sd = torch.stack([ops.scan_state_pack(r.reshape(heads, n_state, head_dim)) for r in state]).to(DEV)
    assert sd.shape[1] == dev_elems
    at = [0, 7, 100]
    for q_lens in ([700, 1, 513], [1, 1, 300]):
        n = sum(q_lens)
        xbc, dt = (torch.randn(n, width) * 0.5).to(dtype), (torch.randn(n, heads) - 1).to(dtype)
        gb, cb = _both(q_lens, at, [0, 1, 2])
        got = ops.selective_scan(xbc.to(DEV), dt.to(DEV), *args, sd, gb, heads, head_dim, n_state, groups)
        want = cpu_ops.selective_scan(xbc.float(), dt.float(), dt_bias, a_log, d_skip, state, cb, heads, head_dim, n_state, groups)
        torch.testing.assert_close(got.cpu(), want, rtol=3e-4, atol=3e-4)
        for slot in range(3):
            torch.testing.assert_close(ops.scan_state_unpack(sd[slot].cpu(), heads, head_dim, n_state).reshape(-1), state[slot], rtol=3e-4, atol=3e-4)
        at = [a + q for a, q in zip(at, q_lens)]


def test_sigmoid_mul_and_cast():
    from cwm_amd import ops

    torch.manual_seed(0)
    for dtype in (torch.float32, torch.bfloat16):
        a, g = torch.randn(5, 77).to(DEV, dtype), torch.randn(5, 90).to(DEV, dtype)
        _close(ops.sigmoid_mul(a, g[:, 4:81]), cpu_ops.sigmoid_mul(a.cpu(), g[:, 4:81].cpu()), dtype, "gate")
    h = torch.randn(4, 33, device=DEV)
    assert ops.cast_rows(h, torch.float32) is h
    assert torch.equal(ops.cast_rows(h, torch.bfloat16), h.to(torch.bfloat16))


@pytest.mark.parametrize("n_experts,top", [(8, 4), (5, 1), (16, 16), (64, 6), (3, 3)])
def test_route_top(n_experts, top):
    from cwm_amd import ops

    torch.manual_seed(n_experts)
    logits = torch.randn(37, n_experts)
    logits[3, :] = 0.25  # all equal: the lower indices win
    chosen, weights = ops.route_top(logits.to(DEV), top)
    want_c, want_w = cpu_ops.route_top(logits, top)
    assert torch.equal(chosen.cpu(), want_c)
    torch.testing.assert_close(weights.cpu(), want_w, rtol=1e-5, atol=1e-6)
    assert chosen[3].tolist() == list(range(top))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_tokens,dim,hidden,n_experts,top", [(1, 64, 32, 8, 4), (9, 176, 88, 6, 4), (200, 72, 40, 3, 2), (300, 64, 50, 4, 1), (33, 100, 36, 16, 3), (1200, 64, 48, 2, 1), (700, 40, 72, 3, 2), (1300, 128, 64, 2, 2), (900, 256, 200, 3, 1), (20, 50, 30, 4, 2)])
def test_routed_experts_pipeline(dtype, n_tokens, dim, hidden, n_experts, top):
    """Grouping, both grouped products and the weighted sum, against one product per pair; sizes that are no
    multiple of a lane's piece take the kernels' element-wise loads."""
    from cwm_amd import ops

    torch.manual_seed(n_tokens + dim)
    x = torch.randn(n_tokens, dim).to(dtype)
    gate, up = (torch.randn(n_experts, hidden, dim) * dim ** -0.5).to(dtype), (torch.randn(n_experts, hidden, dim) * dim ** -0.5).to(dtype)
    down = (torch.randn(n_experts, dim, hidden) * hidden ** -0.5).to(dtype)
    logits = torch.randn(n_tokens, n_experts)
    chosen, weights = cpu_ops.route_top(logits, top)
    rows = cpu_ops.grouped_gate_up(x.float(), chosen, gate.float(), up.float())
    want = cpu_ops.combine_routed(cpu_ops.grouped_linear(rows.to(dtype).float(), chosen, down.float()), chosen, weights)
    groups = ops.group_by_expert(chosen.to(DEV), n_experts)
    # every pair has a row of its expert's tiles, and no row is used twice
    pair_row, row_token, tile_expert = groups.pair_row.cpu(), groups.row_token.cpu(), groups.tile_expert.cpu()
    assert len(set(pair_row.tolist())) == n_tokens * top and int(pair_row.min()) >= 0
    for pair, row in enumerate(pair_row.tolist()):
        assert int(row_token[row]) == pair // top and int(tile_expert[row // 16]) == int(chosen.reshape(-1)[pair])
    hidden_rows = ops.grouped_gate_up(x.to(DEV), groups, gate.to(DEV), up.to(DEV))
    out = ops.combine_routed(ops.grouped_linear(hidden_rows, groups, down.to(DEV)), groups, weights.to(DEV))
    tol = dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    torch.testing.assert_close(out.cpu(), want, **tol)
    # a token's result does not depend on the rest of the step: the same bits beside other tokens (as long as the step
    # takes the same shape of block; a step of many more rows an expert takes another and differs by rounding)
    def through(n):
        g = ops.group_by_expert(chosen[:n].to(DEV), n_experts)
        rows_n = ops.grouped_gate_up(x[:n].to(DEV), g, gate.to(DEV), up.to(DEV))
        return ops.combine_routed(ops.grouped_linear(rows_n, g, down.to(DEV)), g, weights[:n].to(DEV))

    alone = through(1)
    assert torch.equal(alone[0], through(min(3, n_tokens))[0])
    torch.testing.assert_close(alone[0], out[0], **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n_tokens,heads,lead,d,n", [(1, 5, 16, 64, 96), (70, 3, 8, 24, 40), (5, 2, 6, 10, 30), (130, 4, 0, 32, 16), (300, 2, 16, 64, 80)])
def test_products_per_head(dtype, n_tokens, heads, lead, d, n):
    from cwm_amd import ops

    torch.manual_seed(heads + d)
    q = torch.randn(n_tokens, heads, lead + d).to(dtype)
    w = (torch.randn(heads, n, d) * d ** -0.5).to(dtype)
    _close(ops.absorb_queries(q.to(DEV), lead, w.to(DEV)), cpu_ops.absorb_queries(q.float(), lead, w.float()), dtype, "absorb")
    _close(ops.expand_values(q.to(DEV), lead, w.to(DEV)), cpu_ops.expand_values(q.float(), lead, w.float()), dtype, "expand")
