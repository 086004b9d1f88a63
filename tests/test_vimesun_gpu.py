"""Vimesun through the step function, the cache manager, the scheduler and the entry point, against the plain
implementation, under every way of cutting the work."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import helpers
from tests import vimesun_cases as cases
from tests.helpers import Request
from tests.plain import vimesun_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = [torch.float32, torch.bfloat16]
DTYPE_IDS = ["fp32", "bf16"]
NAMES = ["P", "Q", "R", "S", "T"]


def _runner(folder, dtype, n_pages=64, max_requests=4, graphs=False):
    from kestrel_amd.engine.loading import load_model, make_runner

    net = load_model(folder, dtype, torch.device("cuda:0"))
    runner = make_runner(net, 16, n_pages, max_requests, enable_graphs=graphs)
    helpers.poison_cache(runner)
    return runner


def _ids(folder, seed, count):
    return helpers.random_ids(seed, count, cases.config_of(folder)["vocab"])


def _expected(folder, ids):
    return plain.forward(cases.config_of(folder), cases.stored_weights(folder), ids)


def _close(got, want, dtype, what):
    """float32: element by element (2e-5). bfloat16: rounding spreads over a row of logits like noise, so the bound is on
    its root mean square over the vocabulary (mean taken off), 4 % of the row's spread, with a cap of 12 % of that
    spread on any single value. Measured on these configurations: 0.9 % on average over the rows, 2.6 % on the worst
    row, which is as far off when its request runs as one whole prompt as when it is decoded token by token. A fault
    of a mechanism moves rows by far more: ``test_a_far_key_and_the_windows_edge_in_the_model`` asks its construction
    for four times the bound, and float32 is held to 2e-5."""
    if dtype == torch.float32:
        return helpers.assert_close(got, want, dtype, what)
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    diff = got - want
    diff = diff - diff.mean(dim=-1, keepdim=True)
    spread = want.std(dim=-1, unbiased=False)
    rms, top = diff.pow(2).mean(dim=-1).sqrt() / spread, diff.abs().max(dim=-1).values / spread
    worst = int(torch.argmax(rms))
    assert bool((rms <= 0.04).all()) and bool((top <= 0.12).all()), \
        f"{what}: row {worst}: rms error {float(rms[worst]):.3g} of the spread, largest {float(top.max()):.3g}"


def _check(folder, dtype, requests, got, what):
    for tag, req in requests.items():
        _close(got[tag], _expected(folder, req.ids), dtype, f"{what} request {tag}")


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_every_layer_run(name, dtype, monkeypatch):
    """The residual stream after every run of a layer (a looped layer counts each time), then the logits."""
    from kestrel_amd.parts import block as block_module
    from kestrel_amd.parts.block import Block

    folder = cases.model_dir(name)
    runner = _runner(folder, dtype)
    ids = _ids(folder, 1, 45)
    seen = []
    original = Block.forward
    monkeypatch.setattr(block_module, "DEFER_RESIDUAL", False)        # every block leaves the stream complete

    def spy(self, x, *args, **kwargs):
        result = original(self, x, *args, **kwargs)
        seen.append(x.detach().double().cpu())
        return result

    Block.forward = spy
    try:
        got = helpers.replay(runner, {"r": Request("r", ids)}, [[("r", len(ids))]])
    finally:
        Block.forward = original
    streams = []
    want = plain.forward(cases.config_of(folder), cases.stored_weights(folder), ids, streams)
    assert len(seen) == len(streams) == len(plain.layer_order(cases.config_of(folder)))
    for run, (a, b) in enumerate(zip(seen, streams)):
        bound = (2e-5 if dtype == torch.float32 else 4e-2) * float(b.abs().max())
        assert float((a - b).abs().max()) <= bound, f"{name} run {run}: {float((a - b).abs().max()):.3g} > {bound:.3g}"
    _close(got["r"], want, dtype, f"{name} logits")


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts(name, dtype):
    """Each request alone and whole: the first tokens of a sequence (1, 2, 3), lengths around a page's and the
    windows' edges, and well beyond every window."""
    folder = cases.model_dir(name)
    runner = _runner(folder, dtype)
    for seed, length in enumerate([1, 2, 3, 7, 8, 16, 17, 33, 40, 41, 51, 120, 260]):
        reqs = {"r": Request("r", _ids(folder, 100 + seed, length))}
        _check(folder, dtype, reqs, helpers.replay(runner, reqs, [[("r", length)]]), f"{name} whole {length}")


@pytest.mark.parametrize("graphs", [False, True], ids=["launched", "graphs"])
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_token_by_token(name, dtype, graphs):
    """Most of the request in one step, then one token a step until every window has passed over decoded tokens
    only; and a request decoded from its very first token."""
    folder = cases.model_dir(name)
    runner = _runner(folder, dtype, graphs=graphs)
    for seed, (length, head) in enumerate([(150, 60), (70, 1), (48, 47)]):
        reqs = {"r": Request("r", _ids(folder, 200 + seed, length))}
        got = helpers.replay(runner, reqs, [[("r", head)]] + [[("r", 1)]] * (length - head))
        _check(folder, dtype, reqs, got, f"{name} decode {length}/{head}")
    assert (runner.graph_replays > 0) == graphs


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_portions_of_changing_size(name, dtype):
    """Portions cut anywhere: in the middle of a page and of a window, down to two tokens."""
    folder = cases.model_dir(name)
    runner = _runner(folder, dtype)
    for seed, cuts in enumerate([[2, 2, 3, 9, 16, 1, 31, 2, 40, 5, 64, 2], [17, 2, 2, 2, 50], [33, 32, 31, 7]]):
        reqs = {"r": Request("r", _ids(folder, 300 + seed, sum(cuts)))}
        _check(folder, dtype, reqs, helpers.replay(runner, reqs, [[("r", c)] for c in cuts]), f"{name} portions {seed}")


@pytest.mark.parametrize("graphs", [False, True], ids=["launched", "graphs"])
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_in_reused_pages_and_slots(name, dtype, graphs):
    """Up to four live requests of unequal lengths, portions of some beside single tokens of others, in a pool so
    small that pages and slots are used again (what is given back is filled with NaN first); every request must
    come out as it does alone."""
    folder = cases.model_dir(name)
    lengths = {"a": 90, "b": 37, "c": 61, "d": 5, "e": 130, "f": 44, "g": 2}
    windowed = all(layer["mixer"].get("mask") for layer in cases.config_of(folder)["layers"])
    runner = _runner(folder, dtype, n_pages=22 if windowed else 24, max_requests=4, graphs=graphs)
    reqs = {tag: Request(tag, _ids(folder, 400 + i, n)) for i, (tag, n) in enumerate(lengths.items())}
    steps = [[("a", 50), ("b", 20)], [("a", 1), ("b", 17), ("c", 30)], [("a", 1), ("c", 2), ("d", 5)],
             [("a", 38), ("c", 29)],                                  # a, c and d end; b ended before
             [("e", 64), ("f", 3)], [("e", 1), ("f", 41), ("g", 2)], [("e", 1)], [("e", 62)], [("e", 1)], [("e", 1)]]
    got = helpers.replay(runner, reqs, steps, poison=True)
    _check(folder, dtype, reqs, got, f"{name} mixed")
    assert runner.cache.free_slots == 4


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_long_decoding_under_graphs(dtype):
    """Three hundred tokens one by one beside a second request that comes and goes: windows slide, pages go back."""
    folder = cases.model_dir("P")
    runner = _runner(folder, dtype, n_pages=12, max_requests=2, graphs=True)
    reqs = {"long": Request("long", _ids(folder, 500, 300)), "short": Request("short", _ids(folder, 501, 25))}
    steps = [[("long", 3)]] + [[("long", 1)]] * 100 + [[("long", 1), ("short", 20)]] + [[("long", 1), ("short", 1)]] * 5 \
        + [[("long", 1)]] * 191
    got = helpers.replay(runner, reqs, steps, poison=True)
    _check(folder, dtype, reqs, got, "long decoding")
    held = max(len([p for p in runner.cache.block_table(g, s) if p >= 0]) for g in range(len(runner.cache.groups))
               for s in runner.cache.live_slots) if runner.cache.live_slots else 0
    assert held == 0


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_a_far_key_and_the_windows_edge_in_the_model(dtype):
    """A token repeated at chosen distances among tokens that are all different: with equal query and key weights (and,
    where kv heads are shared, every query head a copy of its kv head's rows) the repeated token's score stands out,
    so a window that is one token off, or a lost far key, changes the logits far beyond rounding; in a prompt and
    decoded token by token."""
    base = cases.model_dir("P")
    config = cases.config_of(base)
    heads, kv_heads, d = (config["layers"][0]["mixer"][k] for k in ("heads", "kv_heads", "dim"))

    def edit(weights):
        for i in range(len(config["layers"])):
            k = weights[f"l{i}.mix.k"].float().reshape(kv_heads, d, -1) * 4
            weights[f"l{i}.mix.k"] = k.reshape(kv_heads * d, -1).to(torch.bfloat16)
            weights[f"l{i}.mix.q"] = k.repeat_interleave(heads // kv_heads, dim=0).reshape(heads * d, -1).to(torch.bfloat16)

    folder = cases.rewrite(base, edit)
    window = config["layers"][0]["mixer"]["mask"]["size"]
    for distance in (window - 1, window, window + 1, 16, 15, 1):
        ids = list(range(10, 10 + 3 * window))                       # all different
        at = 2 * window + 5
        ids[at] = ids[at - distance]
        want = _expected(folder, ids)
        for head in (len(ids), at - 3):                              # the repeat inside the prompt; decoded alone
            runner = _runner(folder, dtype)
            reqs = {"r": Request("r", ids)}
            got = helpers.replay(runner, reqs, [[("r", head)]] + [[("r", 1)]] * (len(ids) - head))
            _close(got["r"], want, dtype, f"distance {distance}, prompt of {head}")
    # the construction shows: moving the repeat across the window's edge changes that token's logits
    inside, outside = list(range(10, 10 + 3 * window)), list(range(10, 10 + 3 * window))
    inside[at], outside[at] = inside[at - (window - 1)], outside[at - window]
    a, b = _expected(folder, inside)[at], _expected(folder, outside)[at]
    moved = float(((a - b) - (a - b).mean()).pow(2).mean().sqrt() / a.std())
    assert moved > 0.16, f"the construction moves the row by {moved:.3g} of its spread only"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_entry_point(name, dtype):
    """Requests of different lengths submitted together through ``InferenceEngine``: the scheduler cuts prompts into
    portions beside the decoding of the others; with and without graphs, one and two steps in flight."""
    from kestrel_amd import InferenceEngine, RuntimeConfig

    folder = cases.model_dir(name)
    config, weights = cases.config_of(folder), cases.stored_weights(folder)
    prompts = [_ids(folder, 600 + i, n) for i, n in enumerate([5, 17, 33, 70])]
    n_new = 24
    slack = 1e-4 if dtype == "float32" else 8e-2
    for graphs, depth in ((False, 1), (True, 2)):
        engine = InferenceEngine.create_sync(RuntimeConfig(model_path=folder, dtype=dtype, max_batch_size=4, kv_cache_pages=40,
                                                           max_num_batched_tokens=48, enable_graphs=graphs, pipeline_depth=depth))
        try:
            results = engine.generate_batch_sync(prompts, max_new_tokens=n_new, temperature=0.0, stop_ids=())
        finally:
            engine.shutdown_sync()
        for prompt, result in zip(prompts, results):
            assert result.finish_reason == "length" and len(result.tokens) == n_new
            logits = plain.forward(config, weights, list(prompt) + list(result.tokens[:-1]))
            for i, token in enumerate(result.tokens):
                row = logits[len(prompt) - 1 + i]
                gap = float(row.max() - row[token])
                assert gap <= slack * max(1.0, float(row.std())), \
                    f"{name} {dtype} graphs={graphs}: token {i} is {token}, plain gives {int(row.argmax())} ({gap:.3g} better)"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_program(dtype, tmp_path):
    """``bin/trace_run`` on a folder of this architecture: steps from standard input, logits into files, slots and
    pages for four requests used again."""
    folder = cases.model_dir("Q")
    ids = {tag: _ids(folder, 700 + i, n) for i, (tag, n) in enumerate({"a": 40, "b": 9, "c": 70, "d": 3, "e": 21}.items())}
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": ids["a"][:30], "want": [0, 29]}, {"id": "b", "tokens": ids["b"], "want": [8]}], "end": ["b"]},
        {"step": 1, "entries": [{"id": "a", "tokens": ids["a"][30:31], "want": [0]}, {"id": "c", "tokens": ids["c"][:64], "want": []},
                                {"id": "d", "tokens": ids["d"], "want": [0, 1, 2]}, {"id": "e", "tokens": ids["e"][:2], "want": [1]}], "end": ["d"]},
        {"step": 2, "entries": [{"id": "c", "tokens": ids["c"][64:], "want": [5]}, {"id": "a", "tokens": ids["a"][31:], "want": [8]},
                                {"id": "e", "tokens": ids["e"][2:], "want": [18]}], "end": ["a", "c", "e"]},
    ]
    out = tmp_path / "out"
    done = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out),
                           "--max-tokens", "256"], input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                          capture_output=True, timeout=600, cwd=ROOT)
    assert done.returncode == 0, done.stderr[-2000:]
    assert [line for line in done.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2"]
    full = {tag: _expected(folder, seq) for tag, seq in ids.items()}
    wanted = {0: [("a", 0), ("a", 29), ("b", 8)], 1: [("a", 30), ("d", 0), ("d", 1), ("d", 2), ("e", 1)],
              2: [("c", 69), ("a", 39), ("e", 20)]}
    vocab = cases.config_of(folder)["vocab"]
    run_dtype = torch.float32 if dtype == "float32" else torch.bfloat16
    for step, places in wanted.items():
        got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(len(places), vocab))
        want = torch.stack([full[tag][p] for tag, p in places])
        _close(got, want, run_dtype, f"trace step {step}")
