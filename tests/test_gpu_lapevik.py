"""The Lapevik architecture on the GPU against the plain implementation: every regime of the replay driver in both
types with pages and state slots that are used again; single layers that leave one mechanism nearly alone; a
sharp attention over long sequences (one far key, or the key behind a page border, decides a token); first
tokens and long decoding through state and cache; decode steps replayed from graphs; and greedy generation
through the engine, the command line and `bin/trace_run`."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import lapevik, traces
from plain import lapevik_plain

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = {"tiny_p": [1, 6, 21, 70, 130], "tiny_q": [9, 33, 2, 100, 57], "tiny_r": [150, 41, 90]}
PAGE_SIZES = {"whole": 16, "tail": 16, "portions": 8, "mixed": 8}


def requests_for(name, lengths=None):
    vocab = lapevik.get(name)["vocab"]
    return {f"r{i}": traces.random_tokens(13 * i + len(name), n, vocab) for i, n in enumerate(lengths or LENGTHS[name])}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("lapevik")
    return {name: lapevik.make_folder(root, name, seed=5) for name in lapevik.ALL}


@pytest.fixture(scope="module")
def plain_cache():
    return {}


def plain_for(folders, cache, name, dtype):
    if (name, dtype) not in cache:
        cache[name, dtype] = lapevik.expected(folders[name], requests_for(name), dtype)
    return cache[name, dtype]


def run(folder, dtype, steps, requests, vocab, **options):
    from cwm_amd.replay import Replayer

    rep = Replayer(folder, dtype, traces.max_live_tokens(steps), poison_freed_pages=True, **options)
    page_use = traces.PageUse(rep.manager)
    outputs = traces.run_in_process(rep, steps, page_use)
    assert rep.manager.live_requests() == []
    return traces.gather(steps, outputs, {k: len(v) for k, v in requests.items()}, vocab), rep, page_use


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(lapevik.ALL))
@pytest.mark.parametrize("regime", ["whole", "tail", "portions", "mixed"])
def test_replay_regimes(folders, plain_cache, name, dtype, regime):
    requests = requests_for(name)
    vocab = lapevik.get(name)["vocab"]
    steps = {"whole": traces.whole, "tail": traces.tail_one_by_one, "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, max_live=3)}[regime](requests)
    got, rep, page_use = run(folders[name], dtype, steps, requests, vocab, page_size=PAGE_SIZES[regime], max_requests=3 if regime == "mixed" else 16)
    want = plain_for(folders, plain_cache, name, dtype)
    for rid in requests:
        lapevik.check(got[rid], want[rid], dtype, f"{name} {dtype} {regime} {rid}")
    if regime == "mixed":
        for g in rep.manager.groups:
            assert page_use.pages_shared_between_requests(g.index) > 0, f"group {g.index}: no page served two requests"


def single_layer(layer: dict, width: int = 40, vocab: int = 83, groups: int = 2) -> dict:
    return {"architecture": "Lapevik", "vocab": vocab, "width": width, "norm": {"eps": 1e-5, "groups": groups}, "layers": [layer]}


SINGLE_LAYERS = {
    "state_space": lapevik._ssm(2, 10, 6, 2, 5, 4),
    "state_space_one_tap": lapevik._ssm(3, 4, 33, 1, 1, 1),
    "latent_attention": lapevik._attn(4, 8, 4, 6, 12, 10, 0.5, 100.0, 4),
    "latent_attention_unrotated_rest": lapevik._attn(1, 20, 24, 36, 40, 64, 0.15, 3000.0, 6),
    "experts_all": {**lapevik._ssm(1, 4, 2, 1, 1, 2), "mlp": lapevik._moe(12, 4, 4)},
    "experts_one_of_many": {**lapevik._ssm(1, 4, 2, 1, 1, 2), "mlp": lapevik._moe(30, 20, 1)},
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", list(SINGLE_LAYERS))
def test_single_layers(tmp_path, which, dtype):
    """One mechanism at a time between embedding and head: whole prompts against the same tokens in portions and one
    by one, and both against the plain implementation."""
    config = single_layer(SINGLE_LAYERS[which])
    folder = lapevik.make_folder(tmp_path, which, seed=2, config=config)
    requests = {f"r{i}": traces.random_tokens(i + 5, n, config["vocab"]) for i, n in enumerate([37, 5, 64])}
    want = lapevik.expected(folder, requests, dtype)
    for make in (traces.whole, traces.portions, lambda r: traces.tail_one_by_one(r, tail=20)):
        steps = make(requests)
        got, _, _ = run(folder, dtype, steps, requests, config["vocab"], page_size=8)
        for rid in requests:
            lapevik.check(got[rid], want[rid], dtype, f"{which} {dtype} {rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_and_slow_state_over_long_sequences(folders, dtype):
    """tiny_r's softmax is sharp and its decays are slow: a token's result hangs on single keys hundreds of places
    back or just behind a page border, and on what the state took in at the sequence's start.  A prompt of 700
    tokens whole, in portions that end at, before and after page borders, and with its last 150 tokens one by one."""
    name = "tiny_r"
    vocab = lapevik.get(name)["vocab"]
    requests = {"long": traces.random_tokens(99, 700, vocab)}
    want = lapevik.expected(folders[name], requests, dtype)
    portions = lambda r: traces.portions(r, sizes=[64, 63, 65, 2, 126, 1, 31, 33, 128, 17])  # noqa: E731
    for make in (traces.whole, portions, lambda r: traces.tail_one_by_one(r, tail=150)):
        steps = make(requests)
        got, _, _ = run(folders[name], dtype, steps, requests, vocab, page_size=32)
        lapevik.check(got["long"], want["long"], dtype, f"{name} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_wider_layers_and_many_rows(tmp_path, dtype):
    """Width 256 and prompts of 600 and 300 tokens: the kernels' shapes for many rows, whole, in large portions beside
    each other, and with a tail of single tokens."""
    config = lapevik.MEDIUM
    folder = lapevik.make_folder(tmp_path, "medium", seed=9, config=config)
    vocab = config["vocab"]
    requests = {"a": traces.random_tokens(31, 600, vocab), "b": traces.random_tokens(32, 300, vocab)}
    want = lapevik.expected(folder, requests, dtype)
    side_by_side = [
        {"step": 0, "entries": [{"id": "a", "tokens": requests["a"][:290], "want": list(range(290))}, {"id": "b", "tokens": requests["b"][:270], "want": list(range(270))}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": requests["a"][290:], "want": list(range(310))}, {"id": "b", "tokens": requests["b"][270:], "want": list(range(30))}], "end": ["a", "b"]},
    ]
    for steps in (traces.whole(requests), side_by_side, traces.tail_one_by_one(requests, tail=20)):
        got, _, _ = run(folder, dtype, steps, requests, vocab, page_size=32)
        for rid in requests:
            lapevik.check(got[rid], want[rid], dtype, f"medium {dtype} {rid}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decoding(folders, dtype):
    """Every token a step of its own from an empty cache and a zero state, for 300 steps."""
    name = "tiny_p"
    vocab = lapevik.get(name)["vocab"]
    requests = {"a": traces.random_tokens(4, 300, vocab)}
    steps = traces.tail_one_by_one(requests, tail=299)
    got, _, _ = run(folders[name], dtype, steps, requests, vocab, page_size=16)
    lapevik.check(got["a"], lapevik.expected(folders[name], requests, dtype)["a"], dtype, f"{name} {dtype} one by one")


def test_a_state_slot_that_is_used_again_starts_from_zero(folders):
    """One slot only: the second request finds the first one's state and cache rows and must not read them."""
    name = "tiny_q"
    vocab = lapevik.get(name)["vocab"]
    a, b = traces.random_tokens(1, 40, vocab), traces.random_tokens(2, 25, vocab)
    both = [
        {"step": 0, "entries": [{"id": "a", "tokens": a, "want": [39]}], "end": ["a"]},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:10], "want": list(range(10))}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[10:], "want": list(range(15))}], "end": ["b"]},
    ]
    got, rep, _ = run(folders[name], "float32", both, {"a": a, "b": b}, vocab, page_size=8, max_requests=1)
    alone, _, _ = run(folders[name], "float32", both[1:], {"b": b}, vocab, page_size=8, max_requests=1)
    assert np.array_equal(got["b"], alone["b"])
    lapevik.check(got["b"], lapevik.expected(folders[name], {"b": b}, "float32")["b"], "float32", "second user of the slot")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_replayed_from_graphs_give_the_same_bits(folders, dtype):
    name = "tiny_q"
    vocab = lapevik.get(name)["vocab"]
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
    config, weights = lapevik.read_folder(folder)
    toks, out = list(prompt), []
    for _ in range(n_new):
        logits = lapevik_plain.forward(weights, config, toks, torch.float64)[-1]
        out.append(int(torch.argmax(logits)))
        toks.append(out[-1])
    return out


@pytest.mark.parametrize("name", ["tiny_p", "tiny_q"])
def test_greedy_generation_through_the_engine(folders, name):
    """The engine's own entry point: scheduler, portions of 24 tokens, continuous batching, sampling kernel; then a
    cache that holds barely more than the longest request, so that requests wait for one another's pages and slots."""
    from cwm_amd.engine import Engine, GenArgs

    vocab = lapevik.get(name)["vocab"]
    prompts = [traces.random_tokens(20 + i, n, vocab) for i, n in enumerate([5, 17, 33, 64])]
    engine = Engine.from_folder(folders[name], GenArgs(use_sampling=False, max_batch=4, max_seq=2048, cache_block=16, max_prefill=24), dtype="float32")
    got = engine.generate_tokens(prompts, max_gen=12)
    for p, g in zip(prompts, got):
        assert g == plain_greedy(folders[name], p, 12)
    small = Engine.from_folder(folders[name], GenArgs(use_sampling=False, max_batch=4, max_seq=96, cache_block=4, max_prefill=24), dtype="float32")
    assert small.generate_tokens(prompts, max_gen=12) == got


def test_command_line_and_trace_run_as_child_processes(folders, tmp_path):
    name = "tiny_p"
    vocab = lapevik.get(name)["vocab"]
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
        want = lapevik.expected(folders[name], requests, dtype)
        for rid in requests:
            lapevik.check(got[rid], want[rid], dtype, f"trace_run {dtype} {rid}")
