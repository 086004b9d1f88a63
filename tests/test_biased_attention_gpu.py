"""The mechanisms of attention with a distance bias, a sink, a window and values of a size of their own, and the
small kernels around it, each alone against the plain implementation's function of the same name."""

import math
from types import SimpleNamespace

import pytest
import torch

from tests.plain import vimesun_plain as plain

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
PAGE = 16


class Case:
    """Rows of keys and values in a paged cache with shuffled pages, and packed queries of those rows."""

    def __init__(self, dtype, heads, kv_heads, d, dv, lengths, starts, window, seed=0, queries=None):
        gen = torch.Generator().manual_seed(seed)
        self.dtype, self.heads, self.kv_heads, self.d, self.dv, self.window = dtype, heads, kv_heads, d, dv, window
        self.lengths, self.starts = lengths, starts
        n_pages = sum(-(-n // PAGE) for n in lengths) + 3
        order = torch.randperm(n_pages, generator=gen).tolist()
        self.k_rows = [plain.unit_rms(torch.randn(n, kv_heads, d, generator=gen, dtype=torch.float64), 0.0) for n in lengths]
        self.v_rows = [torch.randn(n, kv_heads, dv, generator=gen, dtype=torch.float64) for n in lengths]
        self.q_rows = [plain.unit_rms(torch.randn(n - s, heads, d, generator=gen, dtype=torch.float64), 0.0)
                       for n, s in zip(lengths, starts)]
        if queries is not None:
            queries(self)
        # what the kernels see is what the storage type keeps
        rnd = lambda t: t.to(dtype).to(torch.float64)
        self.k_rows, self.v_rows, self.q_rows = [rnd(t) for t in self.k_rows], [rnd(t) for t in self.v_rows], [rnd(t) for t in self.q_rows]
        k_cache = torch.full((n_pages, kv_heads, PAGE, d), float("nan"), dtype=torch.float64)
        v_cache = torch.full((n_pages, kv_heads, dv, PAGE), float("nan"), dtype=torch.float64)
        max_pages = max(-(-n // PAGE) for n in lengths) + 1
        table = torch.full((len(lengths), max_pages), -1, dtype=torch.int32)
        for r, n in enumerate(lengths):
            for p in range(-(-n // PAGE)):
                page = order.pop()
                table[r, p] = page
                keys = slice(p * PAGE, min(n, (p + 1) * PAGE))
                count = keys.stop - keys.start
                k_cache[page, :, :count] = self.k_rows[r][keys].transpose(0, 1)
                v_cache[page, :, :, :count] = self.v_rows[r][keys].permute(1, 2, 0)
        # pages that a window has passed are given back: the table then says -1
        if window is not None:
            for r, (n, s) in enumerate(zip(lengths, starts)):
                for p in range(max(0, s + 1 - window) // PAGE):
                    k_cache[table[r, p]] = float("nan")
                    v_cache[table[r, p]] = float("nan")
                    table[r, p] = -1
        token_row, positions, kv_hi, kv_lo, cu_q = [], [], [], [], [0]
        for r, (n, s) in enumerate(zip(lengths, starts)):
            for p in range(s, n):
                token_row.append(r)
                positions.append(p)
                kv_hi.append(p + 1)
                kv_lo.append(0 if window is None else max(0, p + 1 - window))
            cu_q.append(len(token_row))
        as_int = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
        self.token_row, self.positions, self.kv_hi, self.cu_q = as_int(token_row), as_int(positions), as_int(kv_hi), as_int(cu_q)
        self.kv_lo = as_int(kv_lo) if window is not None else None
        self.k_cache, self.v_cache, self.table = k_cache.to(DEV, dtype), v_cache.to(DEV, dtype), table.to(DEV)
        self.q = torch.cat([t.reshape(t.shape[0], heads * d) for t in self.q_rows]).to(DEV, dtype).contiguous()
        self.n = self.q.shape[0]
        self.slopes = torch.tensor(plain.head_slopes(heads), dtype=torch.float32, device=DEV)

    def expected(self, scale):
        out = [plain.attention_core(q, k, v, scale, self.window, range(s, n)).reshape(n - s, self.heads * self.dv)
               for q, k, v, n, s in zip(self.q_rows, self.k_rows, self.v_rows, self.lengths, self.starts)]
        return torch.cat(out)

    def batch(self):
        """What the matrix-core kernel takes from a step: its blocks of 32 queries, or that it is a decode step."""
        decode_only = all(n - s == 1 for n, s in zip(self.lengths, self.starts))
        rows, first = [], []
        for r, (n, s) in enumerate(zip(self.lengths, self.starts)):
            for b in range(0, n - s, 32):
                rows.append(r)
                first.append(int(self.cu_q[r]) + b)
        as_int = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
        return SimpleNamespace(decode_only=decode_only, query_blocks={32: (as_int(rows), as_int(first))}, cu_q=self.cu_q)


def _run(case, scale, kernel):
    from kestrel_amd.ops import core, fast

    out = torch.full((case.n, case.heads * case.dv), float("nan"), dtype=case.dtype, device=DEV)
    if kernel == "generic":
        core.attention_generic(case.q, case.k_cache, case.v_cache, case.table, case.token_row, case.kv_lo, case.kv_hi, out,
                               scale, case.heads, case.kv_heads, case.d, case.dv, case.positions, case.slopes, 0.0)
    else:
        done = fast.attention_biased_bf16(case.q, case.k_cache, case.v_cache, case.table, case.token_row, case.kv_lo,
                                          case.kv_hi, out, scale, case.heads, case.kv_heads, case.d, case.dv,
                                          case.positions, case.slopes, 0.0, case.batch())
        assert done, "the matrix-core kernel declined sizes it is meant to take"
    torch.cuda.synchronize()
    return out.double().cpu()


def _close(got, want, dtype, what):
    atol, rtol = (2e-5, 2e-5) if dtype == torch.float32 else (3e-2, 2e-2)
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    assert bool((err <= bound).all()), f"{what}: max error {float(err.max()):.3g} (bound {float(bound.min()):.3g})"


KERNELS = [("generic", torch.float32), ("generic", torch.bfloat16), ("mfma", torch.bfloat16)]
SIZES = [(4, 2, 32, 64), (8, 1, 48, 32), (2, 2, 64, 64), (4, 1, 128, 128), (6, 3, 96, 112), (3, 1, 32, 20)]


@pytest.mark.parametrize("kernel, dtype", KERNELS, ids=["generic-fp32", "generic-bf16", "mfma-bf16"])
@pytest.mark.parametrize("heads, kv_heads, d, dv", SIZES)
def test_prompts_portions_and_single_tokens_in_one_launch(kernel, dtype, heads, kv_heads, d, dv):
    """Whole prompts, a portion that starts in the middle of a page behind a window's give-back, portions of two and
    of 33 tokens, and single tokens, all in one batch, with and without a window."""
    for window in (None, 40, 7, 1):
        case = Case(dtype, heads, kv_heads, d, dv, lengths=[70, 133, 9, 2, 101, 64, 300], starts=[0, 100, 7, 0, 100, 63, 267],
                    window=window, seed=heads + d)
        _close(_run(case, 0.37, kernel), case.expected(0.37), dtype, f"window {window}")


@pytest.mark.parametrize("kernel, dtype", KERNELS, ids=["generic-fp32", "generic-bf16", "mfma-bf16"])
@pytest.mark.parametrize("heads, kv_heads, d, dv", SIZES + [(32, 1, 32, 32), (40, 1, 32, 64)])
def test_decode_steps(kernel, dtype, heads, kv_heads, d, dv):
    """One token per row (the kernel then puts the heads that share a kv head side by side), rows of very different
    lengths, also a row of one token."""
    lengths = [1, 2, 16, 17, 33, 250, 129, 700]
    for window in (None, 120, 16):
        case = Case(dtype, heads, kv_heads, d, dv, lengths=lengths, starts=[n - 1 for n in lengths], window=window, seed=d + dv)
        assert case.batch().decode_only
        _close(_run(case, 0.21, kernel), case.expected(0.21), dtype, f"window {window}")


def _point_at(distance_of):
    """Queries that all point at one key of their row, chosen by its distance from the query: with a large scale
    the output is that key's value if it is seen and (almost) nothing if it is not, whatever the other keys hold."""
    def edit(case):
        for r, (n, s) in enumerate(zip(case.lengths, case.starts)):
            for i, place in enumerate(range(s, n)):
                j = place - distance_of(place)
                if 0 <= j <= place:
                    for h in range(case.heads):
                        case.q_rows[r][i, h] = case.k_rows[r][j, h // (case.heads // case.kv_heads)]
    return edit


@pytest.mark.parametrize("kernel, dtype", KERNELS, ids=["generic-fp32", "generic-bf16", "mfma-bf16"])
@pytest.mark.parametrize("mode", ["prompt", "decode"])
def test_one_key_that_stands_out(kernel, dtype, mode):
    """A key far back, the last one inside the window, the first one outside it, keys at page borders, the first
    token of the sequence: the query points at it with a score that dwarfs the others'."""
    window, scale, d = 120, 1.5, 32          # a matching key scores 1.5 * 32 = 48, the others around 1.5 * sqrt(32)
    lengths = [400, 277, 150, 121, 120]
    starts = [0] * len(lengths) if mode == "prompt" else [n - 1 for n in lengths]
    for what, distance in (("far", lambda p: p - 3 if window is None else min(p, window - 6)),
                           ("last inside", lambda p: window - 1), ("first outside", lambda p: window),
                           ("page border", lambda p: p % 16 + 1), ("page start", lambda p: p % 16),
                           ("itself", lambda p: 0), ("first token", lambda p: p)):
        case = Case(dtype, 4, 2, d, 64, lengths, starts, window, seed=3, queries=_point_at(distance))
        got, want = _run(case, scale, kernel), case.expected(scale)
        _close(got, want, dtype, f"{mode} {what}")
        # the case shows what it is meant to: where the key is seen the output is its value, else far from it
        at = 0
        for r, (n, s) in enumerate(zip(lengths, starts)):
            for place in range(s, n):
                j = place - distance(place)
                if 0 <= j <= place and what != "first outside" and place - j < window:
                    last_head = want[at, 3 * 64:]          # (the head of the gentlest slope: distance costs it little)
                    assert float((last_head - case.v_rows[r][j, 1]).abs().max()) < 0.05, (what, place)
                at += 1


@pytest.mark.parametrize("kernel, dtype", KERNELS, ids=["generic-fp32", "generic-bf16", "mfma-bf16"])
def test_the_sink_takes_what_the_keys_leave(kernel, dtype):
    """Scores far below the sink's: the weights add up to almost nothing and so does the output; scores far above:
    the sink does not matter. A negative scale makes every score negative by the queries' own keys."""
    case = Case(dtype, 4, 2, 32, 64, [50, 20], [0, 19], 30, seed=5, queries=_point_at(lambda p: 0))
    low = _run(case, -1.0, kernel)              # its own key scores -32, the others about -5: weights of e^-5 and less
    _close(low, case.expected(-1.0), dtype, "low scores")
    case = Case(dtype, 4, 2, 32, 64, [50, 20], [0, 19], 30, seed=5, queries=_point_at(lambda p: 0))
    _close(_run(case, 1.0, kernel), case.expected(1.0), dtype, "high scores")
    # a lone first token with a weak score: half the weight goes to the sink (score 0 against score 0)
    case = Case(dtype, 2, 1, 32, 32, [1], [0], None, seed=6)
    got = _run(case, 0.0, kernel)
    _close(got, 0.5 * case.v_rows[0][0, 0].repeat(2).reshape(1, -1), dtype, "half to the sink")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_unit_norm_and_cache_write(dtype):
    from kestrel_amd.ops import core

    torch.manual_seed(1)
    heads, kv_heads, d, dv, n, eps = 5, 2, 24, 40, 37, 1e-3
    qkv = (torch.randn(n, (heads + kv_heads) * d + kv_heads * dv) * 3).to(dtype)
    pages = 6
    slots = torch.randperm(pages * PAGE)[:n].to(torch.int32)
    slots[5] = -1                                          # a token that is cached nowhere
    k_cache = torch.zeros(pages, kv_heads, PAGE, d, dtype=dtype, device=DEV)
    v_cache = torch.zeros(pages, kv_heads, dv, PAGE, dtype=dtype, device=DEV)
    dev = qkv.to(DEV).clone()
    core.unit_norm_cache(dev, slots.to(DEV), k_cache, v_cache, heads, kv_heads, d, dv, PAGE, eps)
    torch.cuda.synchronize()
    x = qkv.double()
    want_qk = plain.unit_rms(x[:, :(heads + kv_heads) * d].reshape(n, heads + kv_heads, d), eps)
    got = dev.double().cpu()
    tol = 1e-6 if dtype == torch.float32 else 1e-2
    assert torch.allclose(got[:, :(heads + kv_heads) * d].reshape(n, -1, d), want_qk, atol=tol, rtol=tol)
    assert torch.equal(got[:, (heads + kv_heads) * d:], x[:, (heads + kv_heads) * d:])         # values pass unchanged
    for t in range(n):
        if int(slots[t]) < 0:
            continue
        page, off = int(slots[t]) // PAGE, int(slots[t]) % PAGE
        assert torch.allclose(k_cache[page, :, off].double().cpu(), want_qk[t, heads:], atol=tol, rtol=tol)
        assert torch.equal(v_cache[page, :, :, off].double().cpu(), x[t, (heads + kv_heads) * d:].reshape(kv_heads, dv))
    assert float(k_cache.abs().sum(dim=(1, 3)).ne(0).sum()) == n - 1
    # the same tokens cut into runs: 16 tokens that fill a page in order leave as the page's block, the others one by one
    ordered = torch.cat([torch.arange(32, 48), torch.tensor([5, 70, 71, 3]), torch.arange(80, 96), torch.tensor([20])]).to(torch.int32)
    first = torch.tensor([0, 16, 20, 36, 37], dtype=torch.int32)          # (the last run is empty: a list of fixed length)
    count = torch.tensor([16, 4, 16, 1, 0], dtype=torch.int32)
    k2, v2 = torch.zeros_like(k_cache), torch.zeros_like(v_cache)
    dev2 = qkv.to(DEV).clone()
    core.unit_norm_cache(dev2, ordered.to(DEV), k2, v2, heads, kv_heads, d, dv, PAGE, eps, runs=(first.to(DEV), count.to(DEV)))
    k3, v3 = torch.zeros_like(k_cache), torch.zeros_like(v_cache)
    dev3 = qkv.to(DEV).clone()
    core.unit_norm_cache(dev3, ordered.to(DEV), k3, v3, heads, kv_heads, d, dv, PAGE, eps)
    torch.cuda.synchronize()
    # (bf16 with runs takes the form that moves 16 bytes a lane: its sums run in another order, a last bit may differ)
    assert torch.equal(v2, v3) and float(v2.abs().sum()) > 0
    assert torch.allclose(k2.float(), k3.float(), atol=tol, rtol=tol) and torch.allclose(dev2.float(), dev3.float(), atol=tol, rtol=tol)
    assert torch.allclose(dev2.double().cpu()[:, :(heads + kv_heads) * d].reshape(n, -1, d), want_qk, atol=tol, rtol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_two_norms_in_one_pass_and_the_weighted_sum(dtype):
    from kestrel_amd.ops import core

    torch.manual_seed(2)
    n, dim, eps = 19, 100, 1e-4
    x = torch.randn(n, dim) * 2 + 0.5
    delta = torch.randn(n, dim)
    g1, b1, g2, b2 = (torch.randn(dim) for _ in range(4))
    xd, dd = x.to(DEV), delta.to(DEV)
    out1 = torch.empty(n, dim, dtype=dtype, device=DEV)
    out2 = torch.empty(n, dim, dtype=dtype, device=DEV)
    core.layernorm_pair(xd, (g1.to(DEV), b1.to(DEV), eps), (g2.to(DEV), b2.to(DEV), eps), out1, out2, delta=dd, scale=0.45, apply=True)
    torch.cuda.synchronize()
    summed = x.double() + 0.45 * delta.double()
    assert torch.allclose(xd.double().cpu(), summed, atol=1e-6) and float(dd.abs().max()) == 0.0
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert torch.allclose(out1.double().cpu(), plain.layer_norm(summed, g1.double(), b1.double(), eps), atol=tol, rtol=tol)
    assert torch.allclose(out2.double().cpu(), plain.layer_norm(summed, g2.double(), b2.double(), eps), atol=tol, rtol=tol)
    # one norm, nothing added; then the sum alone
    dd.fill_(3.0)
    core.layernorm_pair(xd, (g1.to(DEV), None, eps), None, out1, None, delta=dd)
    assert torch.allclose(out1.double().cpu(), plain.layer_norm(summed, g1.double(), torch.zeros(dim, dtype=torch.float64), eps), atol=tol, rtol=tol)
    assert float(dd.abs().max()) == 0.0 and torch.allclose(xd.double().cpu(), summed, atol=1e-6)
    dd.copy_(delta)
    core.add_scaled(xd, dd, -0.45)
    assert torch.allclose(xd.double().cpu(), x.double(), atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_position_rows_and_streams_side_by_side(dtype):
    from kestrel_amd.ops import core

    torch.manual_seed(3)
    n, dim = 11, 36
    table = torch.randn(50, dim).to(dtype)
    places = torch.tensor([0, 49, 7, 7, 3, 50, 12, 1, 2, 48, 5], dtype=torch.int32)      # (50: outside the table)
    x = torch.randn(n, dim)
    xd = x.to(DEV)
    core.add_table_rows(table.to(DEV), places.to(DEV), xd)
    want = x.clone()
    for t, p in enumerate(places.tolist()):
        if p < 50:
            want[t] += table[p].float()
    assert torch.allclose(xd.cpu(), want, atol=1e-6)
    both = torch.zeros(n, 2 * dim, dtype=dtype, device=DEV)
    other = torch.randn(n, dim, device=DEV)
    core.cast_columns(xd, both[:, :dim])
    core.cast_columns(other, both[:, dim:])
    assert torch.equal(both.cpu(), torch.cat([xd, other], dim=1).to(dtype).cpu())


@pytest.mark.parametrize("rows", [1, 7, 40, 300])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_relu_squared_in_every_linear_kernel(rows, dtype):
    """Few rows go to the weight-streaming kernels, many to the tiled ones (the vendor library has no such epilogue and
    hands the case on)."""
    from kestrel_amd.ops.linear import activation_code, linear

    torch.manual_seed(rows)
    k, n = 96, 152
    a = torch.randn(rows, k).to(dtype)
    w = (torch.randn(n, k) * 0.2).to(dtype)
    out = torch.empty(rows, n, dtype=dtype, device=DEV)
    linear(a.to(DEV), w.to(DEV), None, out, act=activation_code("relu_squared"))
    want = torch.relu(a.double() @ w.double().T) ** 2
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    assert torch.allclose(out.double().cpu(), want, atol=tol * float(want.abs().max()), rtol=tol)
