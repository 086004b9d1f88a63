"""Plain implementation of the Bogivik decoder: float64, whole sequences, no cache, one function per mechanism.

It shares no code with the package: it reads the ``config.json`` dictionary and the stored tensors by their names.
For tokens ``t_0 .. t_{n-1}`` at places ``0 .. n-1``:

* ``x = embed[t_p]``
* a layer ``i``: ``h = rms(x; norm1)``, ``x <- x + mixer(h) + ff(h)`` (one norm, both branches read it; ``ff`` may be absent)
* mixer ``attention``: grouped heads, queries and keys normalised over their whole projection, a query factor that grows
  with the place, a learned bias per bucket of distance and head, softmax over all ``j <= i``, values blended with those of
  the first blending layer, an output gate
* mixer ``parallel``: the mean of two normalised branches, chunked rotary attention (left) and a gated matrix memory (right)
* ``ff``: ``down(gelu_tanh(gate h) * (up h))``
* logits ``head @ rms(x; final.norm)``.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

F64 = torch.float64


def rms_norm(x: torch.Tensor, gain: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps)`` over the last axis, times ``gain`` if there is one."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if gain is None else y * gain


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def gated_mlp(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str) -> torch.Tensor:
    return (gelu_tanh(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


# ---------------------------------------------------------------------------------------------- rotation
def rotary_frequencies(rot: dict) -> List[float]:
    """``f_i = base ** (-2 i / dims)``, rescaled by wavelength where ``rot`` has a ``scaling``: kept below
    ``original / high``, divided by ``factor`` above ``original / low``, blended linearly in between."""
    dims, base = rot["dims"], float(rot["base"])
    out = []
    scaling = rot.get("scaling")
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f = f / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate_pairs(x: torch.Tensor, places: Sequence[int], freqs: Sequence[float]) -> torch.Tensor:
    """``x`` ``[n, heads, d]``: channels ``2 i`` and ``2 i + 1`` of every head turn by ``place * freqs[i]``; channels
    behind ``2 len(freqs)`` stay."""
    out = x.clone()
    p = torch.tensor(list(places), dtype=F64)[:, None]
    for i, f in enumerate(freqs):
        c, s = torch.cos(p * f), torch.sin(p * f)
        u, v = x[:, :, 2 * i], x[:, :, 2 * i + 1]
        out[:, :, 2 * i] = u * c - v * s
        out[:, :, 2 * i + 1] = v * c + u * s
    return out


# ---------------------------------------------------------------------------------------------- softmax attention
def softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, seen: torch.Tensor,
                      bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``q`` ``[nq, H, d]``, ``k`` ``[nk, G, d]``, ``v`` ``[nk, G, dv]``, ``seen`` bool ``[nq, nk]``, ``bias`` ``[H, nq, nk]``
    added to the scaled scores. Returns ``[nq, H, dv]``."""
    nq, n_heads, _ = q.shape
    n_kv, dv = v.shape[1], v.shape[2]
    out = torch.zeros(nq, n_heads, dv, dtype=F64)
    for h in range(n_heads):
        g = h // (n_heads // n_kv)
        scores = (q[:, h] @ k[:, g].T) * scale
        if bias is not None:
            scores = scores + bias[h]
        scores = scores.masked_fill(~seen, -math.inf)
        out[:, h] = torch.softmax(scores, dim=-1) @ v[:, g]
    return out


def causal_mask(n: int) -> torch.Tensor:
    i = torch.arange(n)
    return i[:, None] >= i[None, :]


def chunk_mask(n: int, size: int) -> torch.Tensor:
    """``j <= i`` within the same chunk of ``size`` places, chunks counted from place 0."""
    i = torch.arange(n)
    return (i[:, None] >= i[None, :]) & ((i[:, None] // size) == (i[None, :] // size))


def distance_bucket(n: int, buckets: int, far: float) -> int:
    """Distances below half the buckets have one each; the rest grow logarithmically up to ``far``."""
    half = buckets // 2
    if n < half:
        return n
    return min(buckets - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (buckets - half))))


def distance_bias(table: torch.Tensor, n: int, far: float) -> torch.Tensor:
    """``table`` ``[buckets, H]`` -> ``[H, n, n]`` with entry ``table[bucket(i - j), h]`` (anything for ``j > i``)."""
    buckets = table.shape[0]
    idx = torch.tensor([[distance_bucket(max(i - j, 0), buckets, far) for j in range(n)] for i in range(n)], dtype=torch.long)
    return table[idx].permute(2, 0, 1)


def query_temperature(n: int, coef: float, every: int) -> torch.Tensor:
    """``1 + coef * ln(floor((p + 1) / every) + 1)`` for places ``0 .. n - 1``."""
    return torch.tensor([1.0 + coef * math.log((p + 1) // every + 1) for p in range(n)], dtype=F64)


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: dict, eps: float, shared: dict) -> torch.Tensor:
    """``shared``: carries the first blending layer's values through the stack (key ``"v_first"``)."""
    n = h.shape[0]
    heads, kv_heads, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm(h @ w[prefix + "q"].T, w[prefix + "q.norm"], eps)
    k = rms_norm(h @ w[prefix + "k"].T, w[prefix + "k.norm"], eps)
    v = h @ w[prefix + "v"].T
    temp = m.get("q_temp")
    if temp:
        q = q * query_temperature(n, float(temp["coef"]), int(temp["every"]))[:, None]
    if m.get("v_mix"):
        if "v_first" in shared:
            lam = w[prefix + "vmix"]
            v = (1.0 - lam) * v + lam * shared["v_first"]
        else:
            shared["v_first"] = v
    bias = distance_bias(w[prefix + "rel"], n, float(m["bias_max"]))
    mixed = softmax_attention(q.view(n, heads, d), k.view(n, kv_heads, d), v.view(n, kv_heads, dv), float(m["scale"]),
                              causal_mask(n), bias)
    gate = torch.sigmoid(h @ w[prefix + "g"].T)
    return (mixed.reshape(n, heads * dv) * gate) @ w[prefix + "o"].T


# ---------------------------------------------------------------------------------------------- the parallel mixer
def chunked_rotary_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    heads, kv_heads, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[prefix + "q"].T + w[prefix + "q.b"]).view(n, heads, d)
    k = (h @ w[prefix + "k"].T + w[prefix + "k.b"]).view(n, kv_heads, d)
    v = (h @ w[prefix + "v"].T + w[prefix + "v.b"]).view(n, kv_heads, dv)
    q = rms_norm(q, w[prefix + "q.norm"], eps)
    k = rms_norm(k, w[prefix + "k.norm"], eps)
    freqs = rotary_frequencies(m["rot"])
    q, k = rotate_pairs(q, range(n), freqs), rotate_pairs(k, range(n), freqs)
    mixed = softmax_attention(q, k, v, float(m["scale"]), chunk_mask(n, int(m["mask"]["size"])))
    gate = torch.sigmoid(h @ w[prefix + "g"].T)
    return (mixed.reshape(n, heads * dv) * gate) @ w[prefix + "o"].T + w[prefix + "o.b"]


def capped(z: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(z / cap)


def matrix_memory(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, log_in: torch.Tensor, log_keep: torch.Tensor,
                  state: Optional[dict] = None) -> torch.Tensor:
    """One head, token by token. ``q``, ``k`` ``[n, d]``, ``v`` ``[n, dv]``, ``log_in``, ``log_keep`` ``[n]``.
    ``m_t = max(keep + m, in)``; ``S_t = exp(keep + m - m_t) S + exp(in - m_t) k v^T``; ``n_t`` the same with ``k``;
    ``o_t = S_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6)``. ``S``, ``n`` and ``m`` start at zero."""
    n, d = k.shape
    dv = v.shape[1]
    S = torch.zeros(d, dv, dtype=F64) if state is None else state["S"]
    nn = torch.zeros(d, dtype=F64) if state is None else state["n"]
    m = torch.zeros((), dtype=F64) if state is None else state["m"]
    out = torch.zeros(n, dv, dtype=F64)
    for t in range(n):
        m_new = torch.maximum(log_keep[t] + m, log_in[t])
        keep, take = torch.exp(log_keep[t] + m - m_new), torch.exp(log_in[t] - m_new)
        S = keep * S + take * torch.outer(k[t], v[t])
        nn = keep * nn + take * k[t]
        m = m_new
        out[t] = (S.T @ q[t]) / (torch.maximum(torch.abs(nn @ q[t]), torch.exp(-m)) + 1e-6)
    if state is not None:
        state.update(S=S, n=nn, m=m)
    return out


def matrix_memory_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    heads, d, dv, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    q = (h @ w[prefix + "q"].T).view(n, heads, d) * d ** -0.5
    k = (h @ w[prefix + "k"].T).view(n, heads, d)
    v = (h @ w[prefix + "v"].T).view(n, heads, dv)
    log_in = capped(h @ w[prefix + "i"].T + w[prefix + "i.b"], cap)
    log_keep = torch.nn.functional.logsigmoid(capped(h @ w[prefix + "f"].T + w[prefix + "f.b"], cap))
    o = torch.stack([matrix_memory(q[:, a], k[:, a], v[:, a], log_in[:, a], log_keep[:, a]) for a in range(heads)], dim=1)
    o = rms_norm(o, None, eps).reshape(n, heads * dv) * w[prefix + "norm"]
    return (o * torch.sigmoid(h @ w[prefix + "g"].T)) @ w[prefix + "o"].T


def parallel_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: dict, eps: float) -> torch.Tensor:
    left = chunked_rotary_attention(h, w, prefix + "left.", m["left"], eps)
    right = matrix_memory_mixer(h, w, prefix + "right.", m["right"], eps)
    return 0.5 * (rms_norm(left, w[prefix + "left.out"], eps) + rms_norm(right, w[prefix + "right.out"], eps))


# ---------------------------------------------------------------------------------------------- the stack
def layer(x: torch.Tensor, w: Dict[str, torch.Tensor], i: int, cfg: dict, shared: dict) -> torch.Tensor:
    eps, spec, p = float(cfg["norm"]["eps"]), cfg["layers"][i], f"l{i}."
    h = rms_norm(x, w[p + "norm1"], eps)
    if spec["type"] == "attention":
        out = attention_mixer(h, w, p + "mix.", spec["mixer"], eps, shared)
    elif spec["type"] == "parallel":
        out = parallel_mixer(h, w, p + "mix.", spec["mixer"], eps)
    else:
        raise ValueError(spec["type"])
    if spec.get("mlp") is not None:
        out = out + gated_mlp(h, w, p + "mlp.")
    return x + out


def forward(cfg: dict, weights: Dict[str, torch.Tensor], ids: Sequence[int], streams: Optional[list] = None) -> torch.Tensor:
    """Logits ``[n, vocab]`` of the whole sequence; ``streams`` (a list) receives the stream after every layer."""
    w = {name: t.to(F64) for name, t in weights.items()}
    x = w["embed"][torch.tensor(list(ids), dtype=torch.long)]
    shared: dict = {}
    for i in range(len(cfg["layers"])):
        x = layer(x, w, i, cfg, shared)
        if streams is not None:
            streams.append(x)
    return rms_norm(x, w["final.norm"], float(cfg["norm"]["eps"])) @ w["head"].T
