"""Bogivik through the step function, the cache manager, the scheduler and the entry point, against the plain
implementation, under every way of cutting the work; and each of its mechanisms' kernels alone."""

import json
import math
import os
import subprocess

import numpy as np
import pytest
import torch

from tests import bogivik_cases as cases
from tests import helpers
from tests.helpers import Request
from tests.plain import bogivik_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = [torch.float32, torch.bfloat16]
DTYPE_IDS = ["fp32", "bf16"]
NAMES = ["P", "Q", "R", "S"]
DEV = "cuda:0"


def _runner(folder, dtype, n_pages=64, max_requests=4, graphs=False):
    from kestrel_amd.engine.loading import load_model, make_runner

    net = load_model(folder, dtype, torch.device(DEV))
    runner = make_runner(net, 16, n_pages, max_requests, enable_graphs=graphs)
    helpers.poison_cache(runner)
    return runner


def _ids(folder, seed, count):
    return helpers.random_ids(seed, count, cases.config_of(folder)["vocab"])


_EXPECTED = {}


def _expected(folder, ids):
    key = (folder, tuple(ids))
    if key not in _EXPECTED:
        _EXPECTED[key] = plain.forward(cases.config_of(folder), cases.stored_weights(folder), ids)
    return _EXPECTED[key]


_NOISY = {}


def _what_rounding_does(folder, ids):
    """Per row of logits, how far the plain implementation itself moves (root mean square over the vocabulary, mean taken
    off, as a share of the row's spread) when every weight is off by a relative 2 ** -8, about what rounding to bfloat16
    does to every intermediate value. The design has places where that is amplified without any fault: the read-out of
    the matrix memory is divided by its own root mean square, so at the first tokens of a sequence, where the memory
    holds one or two outer products, the sign of a single small dot product decides the sign of the whole head."""
    if folder not in _NOISY:
        gen = torch.Generator().manual_seed(99)
        _NOISY[folder] = [{k: (v.double() * (1 + 2.0 ** -8 * torch.randn(v.shape, generator=gen, dtype=torch.float64)))
                           for k, v in cases.stored_weights(folder).items()} for _ in range(3)]
    want = _expected(folder, ids)
    worst = torch.zeros(want.shape[0], dtype=torch.float64)
    for noisy in _NOISY[folder]:          # (a flipped sign happens or does not: the largest of three draws)
        moved = plain.forward(cases.config_of(folder), noisy, ids) - want
        moved = moved - moved.mean(dim=-1, keepdim=True)
        worst = torch.maximum(worst, moved.pow(2).mean(dim=-1).sqrt() / want.std(dim=-1, unbiased=False))
    return worst


def _close(got, want, dtype, what, folder=None, ids=None, rows=None):
    """Row by row: the root mean square of the difference over the vocabulary (mean taken off) as a share of the row's
    spread. float32: 1e-4; bfloat16: 4 %; and on rows where rounding alone is amplified by the design (measured on the
    plain implementation, ``_what_rounding_does``), 0.2 % (float32) and eight times (bfloat16: the largest of three draws is a coarse measure of a flip that happens or not) what that moves the row
    by. No single value may be off by more than four times its row's bound. A fault of a mechanism moves rows by far
    more (the constructions below ask for several times the bound)."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    diff = got - want
    diff = diff - diff.mean(dim=-1, keepdim=True)
    spread = want.std(dim=-1, unbiased=False)
    rms, top = diff.pow(2).mean(dim=-1).sqrt() / spread, diff.abs().max(dim=-1).values / spread
    floor, share = (1e-4, 2e-3) if dtype == torch.float32 else (0.04, 8.0)
    bound = torch.full_like(rms, floor)
    if folder is not None and not bool((rms <= bound).all() and (top <= 4 * bound).all()):
        moved = _what_rounding_does(folder, ids)
        bound = torch.maximum(bound, share * (moved[:len(rms)] if rows is None else moved[list(rows)]))
    worst = int(torch.argmax(rms / bound))
    assert bool((rms <= bound).all()) and bool((top <= 4 * bound).all()), \
        f"{what}: row {worst}: rms error {float(rms[worst]):.3g} of the spread (bound {float(bound[worst]):.3g}), largest {float(top[worst]):.3g}"


def _check(folder, dtype, requests, got, what):
    for tag, req in requests.items():
        _close(got[tag], _expected(folder, req.ids), dtype, f"{what} request {tag}", folder, req.ids)


# ------------------------------------------------------------------------------------------------ the model, cut every way
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_every_layer(name, dtype):
    """The residual stream after every layer, then the logits."""
    from kestrel_amd.parts.block import Block

    folder = cases.model_dir(name)
    runner = _runner(folder, dtype)
    ids = _ids(folder, 1, 45)
    seen = []
    original = Block.forward

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
    assert len(seen) == len(streams)
    for layer, (a, b) in enumerate(zip(seen, streams)):
        # nine rows in ten (the rest may be rows where the design amplifies rounding, see ``_what_rounding_does``)
        per_row = (a - b).abs().max(dim=1).values
        bound = (1e-4 if dtype == torch.float32 else 6e-2) * float(b.abs().max())
        assert float(per_row.quantile(0.9)) <= bound, f"{name} layer {layer}: {float(per_row.quantile(0.9)):.3g} > {bound:.3g}"
    _close(got["r"], want, dtype, f"{name} logits", folder, ids)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts(name, dtype):
    """Each request alone and whole: the first tokens of a sequence (1, 2, 3), lengths around a page's, a chunk's and a
    period's edges, and well beyond every far distance."""
    folder = cases.model_dir(name)
    runner = _runner(folder, dtype)
    for seed, length in enumerate([1, 2, 3, 7, 8, 16, 17, 24, 25, 33, 48, 49, 65, 120, 260]):
        reqs = {"r": Request("r", _ids(folder, 100 + seed, length))}
        _check(folder, dtype, reqs, helpers.replay(runner, reqs, [[("r", length)]]), f"{name} whole {length}")


@pytest.mark.parametrize("graphs", [False, True], ids=["launched", "graphs"])
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_token_by_token(name, dtype, graphs):
    """Most of the request in one step, then one token a step across chunk edges and far distances; and a request decoded
    from its very first token (the state of the matrix memory starts at zero and is carried through every step)."""
    folder = cases.model_dir(name)
    runner = _runner(folder, dtype, graphs=graphs)
    for seed, (length, head) in enumerate([(150, 60), (70, 1), (48, 47)]):
        reqs = {"r": Request("r", _ids(folder, 200 + seed, length))}
        got = helpers.replay(runner, reqs, [[("r", head)]] + [[("r", 1)]] * (length - head))
        _check(folder, dtype, reqs, got, f"{name} decode {length}/{head}")
    assert (runner.graph_replays > 0) == graphs


@pytest.mark.parametrize("graphs", [False, True], ids=["launched", "graphs"])
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_portions_of_changing_size(name, dtype, graphs):
    """Portions cut anywhere: in the middle of a page and of a chunk, down to two tokens."""
    folder = cases.model_dir(name)
    runner = _runner(folder, dtype, graphs=graphs)
    for seed, cuts in enumerate([[2, 2, 3, 9, 16, 1, 31, 2, 40, 5, 64, 2], [17, 2, 2, 2, 50], [33, 32, 31, 7]]):
        reqs = {"r": Request("r", _ids(folder, 300 + seed, sum(cuts)))}
        _check(folder, dtype, reqs, helpers.replay(runner, reqs, [[("r", c)] for c in cuts]), f"{name} portions {seed}")


@pytest.mark.parametrize("graphs", [False, True], ids=["launched", "graphs"])
@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_in_reused_pages_and_slots(name, dtype, graphs):
    """Up to four live requests of unequal lengths, portions of some beside single tokens of others, in a pool so small
    that pages and state slots are used again (what is given back is filled with NaN first); every request must come
    out as it does alone."""
    folder = cases.model_dir(name)
    lengths = {"a": 90, "b": 37, "c": 61, "d": 5, "e": 130, "f": 44, "g": 2}
    runner = _runner(folder, dtype, n_pages=24, max_requests=4, graphs=graphs)
    reqs = {tag: Request(tag, _ids(folder, 400 + i, n)) for i, (tag, n) in enumerate(lengths.items())}
    steps = [[("a", 50), ("b", 20)], [("a", 1), ("b", 17), ("c", 30)], [("a", 1), ("c", 2), ("d", 5)],
             [("a", 38), ("c", 29)],                                  # a, c and d end; b ended before
             [("e", 64), ("f", 3)], [("e", 1), ("f", 41), ("g", 2)], [("e", 1)], [("e", 62)], [("e", 1)], [("e", 1)]]
    got = helpers.replay(runner, reqs, steps, poison=True)
    _check(folder, dtype, reqs, got, f"{name} mixed")
    assert runner.cache.free_slots == 4


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_long_decoding_under_graphs(dtype):
    """Three hundred tokens one by one beside a second request that comes and goes: chunks pass, their pages go back."""
    folder = cases.model_dir("P")
    runner = _runner(folder, dtype, n_pages=24, max_requests=2, graphs=True)
    reqs = {"long": Request("long", _ids(folder, 500, 300)), "short": Request("short", _ids(folder, 501, 25))}
    steps = [[("long", 3)]] + [[("long", 1)]] * 100 + [[("long", 1), ("short", 20)]] + [[("long", 1), ("short", 1)]] * 5 \
        + [[("long", 1)]] * 191
    got = helpers.replay(runner, reqs, steps, poison=True)
    _check(folder, dtype, reqs, got, "long decoding")
    assert not runner.cache.live_slots


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_a_far_key_and_the_chunks_edge_in_the_model(dtype):
    """A token repeated at chosen distances among tokens that are all different. With equal query and key weights the
    repeated token's score stands out in the attention layers (far keys, whatever bucket they fall into) and in the
    chunked branch (only inside the chunk), and with a forget gate near one the matrix memory keeps it: a chunk that is
    one token off, a lost far key or a lost state changes the logits far beyond rounding; in a prompt and decoded."""
    base = cases.model_dir("P")
    config = cases.config_of(base)

    def edit(weights):
        for i, layer in enumerate(config["layers"]):
            prefix = f"l{i}.mix." + ("left." if layer["type"] == "parallel" else "")
            m = layer["mixer"]["left"] if layer["type"] == "parallel" else layer["mixer"]
            heads, kv_heads, d = m["heads"], m["kv_heads"], m["dim"]
            k = weights[prefix + "k"].float().reshape(kv_heads, d, -1) * 3
            weights[prefix + "k"] = k.reshape(kv_heads * d, -1).to(torch.bfloat16)
            weights[prefix + "q"] = k.repeat_interleave(heads // kv_heads, dim=0).reshape(heads * d, -1).to(torch.bfloat16)
            if layer["type"] == "parallel":
                weights[f"l{i}.mix.right.f.b"] = torch.full_like(weights[f"l{i}.mix.right.f.b"], 5.0)
                weights[f"l{i}.mix.right.q"] = weights[f"l{i}.mix.right.k"].clone()

    folder = cases.rewrite(base, edit)
    chunk = config["layers"][1]["mixer"]["left"]["mask"]["size"]
    length = 4 * chunk
    at = 3 * chunk + 5                                              # the sixth place of the fourth chunk
    for distance in (5, 6, 4, 1, 2 * chunk, at - 1, at):
        ids = list(range(10, 10 + length))                          # all different
        ids[at] = ids[at - distance]
        want = _expected(folder, ids)
        for head in (len(ids), at - 3):                             # the repeat inside the prompt; decoded alone
            runner = _runner(folder, dtype)
            reqs = {"r": Request("r", ids)}
            got = helpers.replay(runner, reqs, [[("r", head)]] + [[("r", 1)]] * (len(ids) - head))
            _close(got["r"], want, dtype, f"distance {distance}, prompt of {head}", folder, ids)
    # the constructions show: moving the repeat across the chunk's edge, or to a far place, changes that token's logits
    def moved(d1, d2):
        one, two = list(range(10, 10 + length)), list(range(10, 10 + length))
        one[at], two[at] = one[at - d1], two[at - d2]
        a, b = _expected(folder, one)[at], _expected(folder, two)[at]
        return float(((a - b) - (a - b).mean()).pow(2).mean().sqrt() / a.std())
    assert moved(5, 6) > 0.16 and moved(2 * chunk, at) > 0.16, (moved(5, 6), moved(2 * chunk, at))


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
                                                           max_num_batched_tokens=48, enable_graphs=graphs, pipeline_depth=depth,
                                                           max_seq_len=128))
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
    """``bin/trace_run`` on a folder of this architecture whose ``config.json`` leaves the number of buckets to the weights
    file: steps from standard input, logits into files, slots and pages for four requests used again."""
    def drop_buckets(config):
        for layer in config["layers"]:
            layer["mixer"].pop("buckets", None)

    folder = cases.rewrite(cases.model_dir("Q"), lambda w: None, drop_buckets)
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
        for row, (tag, p) in enumerate(places):
            _close(got[row:row + 1], want[row:row + 1], run_dtype, f"trace step {step} {tag}[{p}]", folder, ids[tag], rows=[p])


def test_command_line(tmp_path):
    """``python -m kestrel_amd random-weights`` from a configuration of this design, then ``generate`` on the folder."""
    import sys

    env = dict(os.environ, PYTHONPATH=ROOT)
    config = tmp_path / "cfg.json"
    config.write_text(json.dumps(cases.CONFIGS["S"]))
    made = subprocess.run([sys.executable, "-m", "kestrel_amd", "random-weights", "--out", str(tmp_path / "m"), "--config", str(config),
                           "--seed", "5", "--std", "0.08", "--bias-std", "0.5", "--gain-std", "0.2"], capture_output=True, text=True,
                          env=env, cwd=ROOT)
    assert made.returncode == 0, made.stderr
    folder = str(tmp_path / "m")
    prompt = _ids(folder, 990, 9)
    done = subprocess.run([sys.executable, "-m", "kestrel_amd", "generate", "--model-path", folder, "--dtype", "float32",
                           "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "6", "--temperature", "0",
                           "--kv-cache-pages", "8", "--max-seq-len", "64"], capture_output=True, text=True, env=env, cwd=ROOT,
                          timeout=300)
    assert done.returncode == 0, done.stderr
    tokens = json.loads(done.stdout.strip().splitlines()[-1])["tokens"]
    assert len(tokens) == 6
    logits = plain.forward(cases.config_of(folder), cases.stored_weights(folder), prompt + tokens[:-1])
    for i, token in enumerate(tokens):
        row = logits[len(prompt) - 1 + i]
        assert float(row.max() - row[token]) <= 1e-4 * max(1.0, float(row.std())), f"token {i}"


# ------------------------------------------------------------------------------------------------ each mechanism's kernel alone
def _gen(seed):
    return torch.Generator().manual_seed(seed)


def _tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


def test_rms_norm_kernel():
    from kestrel_amd.ops import core

    g = _gen(1)
    for n, dim in ((5, 100), (3, 1024), (1, 7)):
        x = torch.randn(n, dim, generator=g) * 3
        gain = torch.randn(dim, generator=g)
        for dtype in DTYPES:
            out = torch.empty(n, dim, dtype=dtype, device=DEV)
            core.rmsnorm(x.to(DEV), gain.to(DEV), 1e-3, out)
            want = plain.rms_norm(x.double(), gain.double(), 1e-3)
            assert torch.allclose(out.double().cpu(), want, **_tol(dtype))
        rows = torch.tensor([2, 0], dtype=torch.int32, device=DEV)[:min(2, n)] if n > 2 else None
        if rows is not None:
            out = torch.empty(2, dim, dtype=torch.float32, device=DEV)
            core.rmsnorm(x.to(DEV), gain.to(DEV), 1e-3, out, rows)
            assert torch.allclose(out.double().cpu(), plain.rms_norm(x.double(), gain.double(), 1e-3)[[2, 0]], rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("hd, hdv", [(24, 10), (64, 40), (32, 64), (128, 128)])
@pytest.mark.parametrize("scope, pairing, rot", [("head", "interleaved", 12), ("projection", "halves", 0), (None, "interleaved", 24),
                                                   ("head", "halves", 8), ("projection", "interleaved", 24)])
def test_prepare_kernel(scope, pairing, rot, hd, hdv, dtype):
    """Norm with gains over a head or the whole projection, a rotation from frequencies with either pairing, the factor on
    queries, blended values, and the cache write, in a buffer whose rows are wider than q | k | v. (Heads of 32, 64 and 128
    channels: in bf16 the kernel that takes eight channels a lane, with more heads than one pass of it covers.)"""
    from kestrel_amd.ops import core

    g = _gen(2)
    n, H, G, ps, extra = 9, 36 if hd == 64 else 4, 2, 4, 8
    total = (H + G) * hd + G * hdv
    x = (torch.randn(n, total + extra, generator=g) * 2).to(dtype)
    places = torch.tensor([0, 1, 2, 3, 100, 101, 7, 63, 64], dtype=torch.int32)
    slots = torch.tensor([5, 4, 7, 6, 12, 13, -1, 0, 1], dtype=torch.int32)
    per_head = scope == "head"
    q_gain = torch.randn(hd if per_head else H * hd, generator=g) if scope else None
    k_gain = torch.randn(hd if per_head else G * hd, generator=g) if scope else None
    freqs = torch.tensor([0.9 ** i for i in range(rot // 2)], dtype=torch.float32) if rot else None
    other = (torch.randn(n, G * hdv, generator=g)).to(dtype)
    lam = torch.tensor([0.3], dtype=torch.float32)
    eps, coef, every = 1e-4, 0.6, 3
    buf = x.clone().to(DEV)
    k_cache = torch.zeros(4, G, ps, hd, dtype=dtype, device=DEV)
    v_cache = torch.zeros(4, G, hdv, ps, dtype=dtype, device=DEV)
    other_dev = other.clone().to(DEV)
    core.qkv_prepare(buf[:, :total], places.to(DEV), slots.to(DEV), k_cache, v_cache, H, G, hd, hdv, ps, scope,
                     None if q_gain is None else q_gain.to(DEV), None if k_gain is None else k_gain.to(DEV), eps,
                     None if freqs is None else freqs.to(DEV), pairing, (coef, every), "blend", other_dev, lam.to(DEV))
    xd = x.double()
    q, k = xd[:, :H * hd], xd[:, H * hd:(H + G) * hd]
    v = xd[:, (H + G) * hd:total]
    if scope == "head":
        q = plain.rms_norm(q.view(n, H, hd), q_gain.double(), eps)
        k = plain.rms_norm(k.view(n, G, hd), k_gain.double(), eps)
    elif scope == "projection":
        q = plain.rms_norm(q, q_gain.double(), eps).view(n, H, hd)
        k = plain.rms_norm(k, k_gain.double(), eps).view(n, G, hd)
    else:
        q, k = q.view(n, H, hd), k.view(n, G, hd)
    if rot:
        f = freqs.double().tolist()
        if pairing == "interleaved":
            q, k = plain.rotate_pairs(q, places.tolist(), f), plain.rotate_pairs(k, places.tolist(), f)
        else:
            def halves(t):
                # channels i and i + rot / 2 as a pair: bring them side by side, turn, put them back
                order = [c for i in range(rot // 2) for c in (i, i + rot // 2)] + list(range(rot, hd))
                turned = plain.rotate_pairs(t[:, :, order], places.tolist(), f)
                back = torch.empty_like(turned)
                back[:, :, order] = turned
                return back
            q, k = halves(q), halves(k)
    q = q * plain.query_temperature(128, coef, every)[places.long()][:, None, None]
    v = (0.7 * v + 0.3 * other.double()).view(n, G, hdv)
    # (float32: an angle of a hundred radians, rounded to 32 bits as the design computes it, is off by 6e-6, times values of up to ten)
    tol = _tol(dtype) if dtype == torch.bfloat16 else dict(rtol=2e-5, atol=2e-4 if rot else 2e-5)
    got = buf.double().cpu()
    assert torch.allclose(got[:, :H * hd], q.reshape(n, -1), **tol), "queries"
    assert torch.equal(got[:, H * hd:], xd[:, H * hd:]), "keys, values and the columns behind them stay as projected"
    for t in range(n):
        s = int(slots[t])
        if s < 0:
            continue
        assert torch.allclose(k_cache[s // ps, :, s % ps].double().cpu(), k[t], **tol), f"cached key of token {t}"
        assert torch.allclose(v_cache[s // ps, :, :, s % ps].double().cpu(), v[t], **tol), f"cached value of token {t}"
    assert float(k_cache[2, :, 2:].abs().max()) == 0 and float(v_cache[2].abs().max()) == 0     # slots nobody named stay untouched
    # a source layer leaves its values as they are
    src = torch.zeros(n, G * hdv, dtype=dtype, device=DEV)
    buf = x.clone().to(DEV)
    core.qkv_prepare(buf[:, :total], None, None, None, None, H, G, hd, hdv, ps, blend="source", v_other=src)
    assert torch.equal(src.cpu(), x[:, (H + G) * hd:total]) and torch.equal(buf.cpu(), x)


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
def test_gate_and_branches_kernels(dtype):
    from kestrel_amd.ops import core

    g = _gen(3)
    n, dim = 6, 50
    x, gate = torch.randn(n, dim + 8, generator=g).to(dtype), (torch.randn(n, dim + 3, generator=g) * 3).to(dtype)
    xd = x.clone().to(DEV)
    core.gate_mul(xd[:, :dim], gate.to(DEV)[:, 3:])
    want = x[:, :dim].double() * torch.sigmoid(gate[:, 3:].double())
    assert torch.allclose(xd[:, :dim].double().cpu(), want, **_tol(dtype)) and torch.equal(xd[:, dim:].cpu(), x[:, dim:])
    if dtype == torch.float32:
        a, b, base = (torch.randn(n, dim, generator=g) * s for s in (5.0, 0.01, 1.0))
        ga, gb = torch.randn(dim, generator=g), torch.randn(dim, generator=g)
        out = base.clone().to(DEV)
        core.branches_sum(out, a.to(DEV), ga.to(DEV), 0.5, b.to(DEV), gb.to(DEV), 0.25, 1e-5)
        want = base.double() + 0.5 * plain.rms_norm(a.double(), ga.double(), 1e-5) + 0.25 * plain.rms_norm(b.double(), gb.double(), 1e-5)
        assert torch.allclose(out.double().cpu(), want, rtol=2e-5, atol=2e-5)
        out = base.clone().to(DEV)
        core.branches_sum(out, a.to(DEV), None, 2.0, eps=1e-5)
        assert torch.allclose(out.double().cpu(), base.double() + 2.0 * plain.rms_norm(a.double(), None, 1e-5), rtol=2e-5, atol=2e-5)


_MEMORY_SIZES = [(3, 20, 36), (1, 8, 300), (2, 64, 64), (2, 200, 200), (2, 64, 128), (1, 32, 256), (1, 128, 128), (3, 64, 256)]


@pytest.mark.parametrize("heads, d, dv, dtype, passes",
                         [(*size, dtype, False) for size in _MEMORY_SIZES for dtype in DTYPES]
                         + [(*size, torch.bfloat16, True) for size in _MEMORY_SIZES if size[1] in (32, 64, 128) and size[2] in (128, 256)],
                         ids=lambda v: {torch.float32: "fp32", torch.bfloat16: "bf16", True: "three passes", False: "in turn"}.get(v, str(v)))
def test_matrix_memory_kernel(heads, d, dv, dtype, passes):
    """Rows of unequal lengths in one launch, cut into steps (a prompt, portions, single tokens), against the plain
    recurrence over the whole sequence: the state in its slot carries everything; a row without a request writes zeros;
    large gates stay finite through the running maximum. (200 x 200: a state too large for LDS; value heads of 128 and
    256: in bf16 the portions go through the kernel that unrolls the recurrence over chunks of 64 tokens, here with rows
    of less than a chunk, of several chunks and a part, and a state that single tokens have advanced in between.)"""
    from kestrel_amd.ops import core, fast

    assert not passes or fast.matrix_memory_chunks_scratch(64, 1, heads, d, dv), "the three passes do not cover these sizes"
    g = _gen(4)
    lengths = [150, 5, 1, 90]
    cap, eps, scale = 6.0, 1e-5, d ** -0.5
    width = 2 * heads * d + 2 * heads * dv + 5
    data = {r: dict(x=(torch.randn(L, width, generator=g)).to(dtype), pre=torch.randn(L, 2 * heads, generator=g) * 8 + 1.0)
            for r, L in enumerate(lengths)}
    gain = torch.randn(heads * dv, generator=g)
    offsets = (3, 3 + heads * d, 3 + 2 * heads * d, 3 + 2 * heads * d + heads * dv)
    per_head = d * dv + d + 1
    state = torch.full((len(lengths) + 1, heads * per_head), float("nan"), device=DEV)
    slot_of = {0: 2, 1: 0, 2: 3, 3: 1}
    for s in slot_of.values():
        state[s].zero_()

    def want_row(r):
        x, pre = data[r]["x"].double(), data[r]["pre"].double()
        L = x.shape[0]
        q = x[:, offsets[0]:offsets[0] + heads * d].view(L, heads, d) * scale
        k = x[:, offsets[1]:offsets[1] + heads * d].view(L, heads, d)
        v = x[:, offsets[2]:offsets[2] + heads * dv].view(L, heads, dv)
        gate = x[:, offsets[3]:offsets[3] + heads * dv]
        li = plain.capped(pre[:, :heads], cap)
        lf = torch.nn.functional.logsigmoid(plain.capped(pre[:, heads:], cap))
        o = torch.stack([plain.matrix_memory(q[:, a], k[:, a], v[:, a], li[:, a], lf[:, a]) for a in range(heads)], dim=1)
        return plain.rms_norm(o, None, eps).reshape(L, heads * dv) * gain.double() * torch.sigmoid(gate)

    # steps: (row, tokens) lists; rows 0 and 3 in portions and single tokens, a padding row (slot -1) in the middle
    steps = [[(0, 10), (1, 5)], [(0, 1), (None, 3), (2, 1), (3, 2)], [(0, 1), (3, 1)], [(0, 138), (3, 87)]]
    done = {r: 0 for r in data}
    got = {r: [] for r in data}
    for step in steps:
        xs, pres, cu, slots = [], [], [0], []
        for r, count in step:
            if r is None:
                xs.append(torch.randn(count, width, generator=g).to(dtype))
                pres.append(torch.randn(count, 2 * heads, generator=g))
                slots.append(-1)
            else:
                xs.append(data[r]["x"][done[r]:done[r] + count])
                pres.append(data[r]["pre"][done[r]:done[r] + count])
                slots.append(slot_of[r])
            cu.append(cu[-1] + count)
        x = torch.cat(xs).to(DEV)
        out = torch.full((x.shape[0], heads * dv), 7.0, dtype=dtype, device=DEV)
        scratch = torch.full((fast.matrix_memory_chunks_scratch(x.shape[0], len(slots), heads, d, dv),), float("nan"),
                             device=DEV) if passes else None
        core.matrix_memory(x, offsets, torch.cat(pres).to(DEV).contiguous(), state, torch.tensor(cu, dtype=torch.int32, device=DEV),
                           torch.tensor(slots, dtype=torch.int32, device=DEV), gain.to(DEV), out, heads, d, dv, scale, cap, eps,
                           single_tokens=all(count == 1 for _, count in step), chunks=True, scratch=scratch)
        for i, (r, count) in enumerate(step):
            piece = out[cu[i]:cu[i + 1]].double().cpu()
            if r is None:
                assert float(piece.abs().max()) == 0.0
            else:
                got[r].append(piece)
                done[r] += count
    assert bool(torch.isnan(state[len(lengths)]).all())                  # the spare row was never touched
    for r in data:
        want = want_row(r)
        have = torch.cat(got[r])
        bound = 3e-5 if dtype == torch.float32 else 3e-2
        assert float((have - want).abs().max()) <= bound * max(1.0, float(want.abs().max())), \
            f"row {r}: {float((have - want).abs().max()):.3g}"


@pytest.mark.parametrize("dtype", DTYPES, ids=DTYPE_IDS)
@pytest.mark.parametrize("hd, hdv, G, H", [(32, 64, 2, 4), (96, 32, 1, 2), (24, 10, 3, 3)])
def test_attention_with_a_distance_table(hd, hdv, G, H, dtype):
    """The bias by distance in the attention kernels (the generic one in both precisions, the matrix-core one in bf16
    where it takes the sizes): queries of a prompt portion and single decoded queries, keys far beyond the table's last
    entry, at page borders and at the chunk's edge (``kv_lo``). One key's score is made to stand out by the table alone."""
    from kestrel_amd.engine.batch import Workspace
    from kestrel_amd.ops import core, fast

    g = _gen(5)
    ps, n_keys, T = 16, 200, 37
    pages = -(-n_keys // ps)
    k = torch.randn(n_keys, G, hd, generator=g).to(dtype)
    v = torch.randn(n_keys, G, hdv, generator=g).to(dtype)
    table = torch.randn(H, T, generator=g) * 2
    table[:, 20] += 9.0                                       # a key twenty places back stands out by the bias alone
    order = torch.randperm(pages, generator=g)
    k_cache = torch.full((pages, G, ps, hd), float("nan"), dtype=dtype, device=DEV)
    v_cache = torch.full((pages, G, hdv, ps), float("nan"), dtype=dtype, device=DEV)
    for j in range(n_keys):
        k_cache[order[j // ps], :, j % ps] = k[j].to(DEV)
        v_cache[order[j // ps], :, :, j % ps] = v[j].to(DEV)
    block_table = order.to(torch.int32).view(1, pages).to(DEV)
    scale = 0.2

    def want_for(places, lows):
        q = queries.double().view(len(places), H, hd)
        out = torch.zeros(len(places), H, hdv, dtype=torch.float64)
        for i, (p, lo) in enumerate(zip(places, lows)):
            seen = torch.zeros(1, n_keys, dtype=torch.bool)
            seen[0, lo:p + 1] = True
            dist = (p - torch.arange(n_keys)).clamp(0, T - 1)
            bias = table.double()[:, dist].unsqueeze(1)
            out[i] = plain.softmax_attention(q[i:i + 1], k.double(), v.double(), scale, seen, bias)[0]
        return out.reshape(len(places), H * hdv)

    for places, lows, decode in (([130 + i for i in range(40)], [0] * 40, False), ([199], [0], True), ([36], [0], True),
                                 ([100 + i for i in range(33)], [96] * 28 + [128] * 5, False), ([19], [16], True)):
        n = len(places)
        queries = torch.randn(n, H * hd, generator=g).to(dtype)
        # (an output gate, applied in the kernels' epilogues, on every second case; its rows lie in a wider buffer)
        gate = (torch.randn(n, H * hdv + 8, generator=g) * 2).to(dtype).to(DEV)[:, 8:] if len(places) % 2 else None
        want = want_for(places, lows)
        if gate is not None:
            want = want * torch.sigmoid(gate.double().cpu())
        args = dict(token_row=torch.zeros(n, dtype=torch.int32, device=DEV), kv_lo=torch.tensor(lows, dtype=torch.int32, device=DEV),
                    kv_hi=torch.tensor([p + 1 for p in places], dtype=torch.int32, device=DEV))
        pos = torch.tensor(places, dtype=torch.int32, device=DEV)
        out = torch.zeros(n, H * hdv, dtype=dtype, device=DEV)
        core.attention_generic(queries.to(DEV), k_cache, v_cache, block_table, args["token_row"], args["kv_lo"], args["kv_hi"], out,
                               scale, H, G, hd, hdv, pos, None, None, bias_table=table.to(DEV), gate=gate)
        assert torch.allclose(out.double().cpu(), want, **_tol(dtype)), f"generic kernel, places {places[0]}.."
        if dtype == torch.bfloat16 and fast.biased_query_block(hd, hdv):
            from types import SimpleNamespace
            tile = fast.biased_query_block(hd, hdv)
            firsts = list(range(0, n, tile))
            batch = SimpleNamespace(decode_only=decode, cu_q=torch.tensor([0, n], dtype=torch.int32, device=DEV),
                                    query_blocks={tile: (torch.zeros(len(firsts), dtype=torch.int32, device=DEV),
                                                         torch.tensor(firsts, dtype=torch.int32, device=DEV))})
            out = torch.zeros(n, H * hdv, dtype=dtype, device=DEV)
            assert fast.attention_biased_bf16(queries.to(DEV), k_cache, v_cache, block_table, args["token_row"], args["kv_lo"],
                                              args["kv_hi"], out, scale, H, G, hd, hdv, pos, None, None, batch, bias_table=table.to(DEV),
                                              gate=gate)
            assert torch.allclose(out.double().cpu(), want, **_tol(dtype)), f"matrix-core kernel, places {places[0]}.."
