"""Plain implementation of the Vimesun decoder: float64, whole sequences, no cache, one function per mechanism.

It shares no code with the package: it reads the ``config.json`` dictionary and the stored tensors by their names
and computes, for tokens ``t_0 .. t_{n-1}`` at places ``0 .. n-1``:

* ``x0[p] = embed[t_p] + pos[p]``
* the layers in order, the stretch ``loop.start .. loop.stop - 1`` run ``loop.times`` times, each pass starting
  with ``x <- loop.in @ concat(x, x0)``
* a layer ``i``: ``x <- x + residual_mult * (attention(LN(x; norm1)) + mlp(LN(x; norm2)))``
* logits ``head @ LN(x; final.norm)``.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence

import torch

F64 = torch.float64


def layer_norm(x: torch.Tensor, gain: torch.Tensor, shift: torch.Tensor, eps: float) -> torch.Tensor:
    """``(x - mean) / sqrt(mean of squared deviations + eps) * gain + shift`` over the last axis."""
    mean = x.mean(dim=-1, keepdim=True)
    dev = x - mean
    return dev / torch.sqrt((dev * dev).mean(dim=-1, keepdim=True) + eps) * gain + shift


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps)`` over the last axis, no gain."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def head_slopes(n_heads: int) -> List[float]:
    """Slope of head ``h``: ``2 ** (-8 (h + 1) / n_heads)``."""
    return [2.0 ** (-8.0 * (h + 1) / n_heads) for h in range(n_heads)]


def sink_softmax_weights(scores: torch.Tensor) -> torch.Tensor:
    """``exp(s_j) / (1 + sum_j exp(s_j))`` over the last axis; ``-inf`` scores weigh nothing. Computed from a
    reference point so that large scores do not overflow."""
    ref = torch.clamp(scores.max(dim=-1, keepdim=True).values, min=0.0)
    e = torch.exp(scores - ref)
    return e / (torch.exp(-ref) + e.sum(dim=-1, keepdim=True))


def attention_core(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: Optional[int],
                   q_places: Optional[Sequence[int]] = None) -> torch.Tensor:
    """``q`` ``[nq, H, d]``, ``k`` ``[nk, G, d]``, ``v`` ``[nk, G, dv]`` (already normalised where they are to be);
    key ``j`` stands at place ``j``, query ``i`` at ``q_places[i]`` (default: ``i``). Returns ``[nq, H, dv]``.
    Query at place ``i`` sees ``0 <= i - j < window`` (``None``: every ``j <= i``)."""
    nq, n_heads, _ = q.shape
    nk, n_kv, dv = v.shape
    places = torch.tensor(list(range(nq)) if q_places is None else list(q_places), dtype=F64)
    dist = places[:, None] - torch.arange(nk, dtype=F64)[None, :]
    seen = dist >= 0
    if window is not None:
        seen &= dist < window
    out = torch.zeros(nq, n_heads, dv, dtype=F64)
    slopes = head_slopes(n_heads)
    for h in range(n_heads):
        g = h // (n_heads // n_kv)
        scores = (q[:, h] @ k[:, g].T) * scale - slopes[h] * dist
        scores = scores.masked_fill(~seen, -math.inf)
        out[:, h] = sink_softmax_weights(scores) @ v[:, g]
    return out


def attention(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, mixer: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    heads, kv_heads, d, dv = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    q = (h @ w[prefix + "q"].T).view(n, heads, d)
    k = (h @ w[prefix + "k"].T).view(n, kv_heads, d)
    v = (h @ w[prefix + "v"].T).view(n, kv_heads, dv)
    window = mixer["mask"]["size"] if mixer.get("mask") else None
    mixed = attention_core(unit_rms(q, eps), unit_rms(k, eps), v, mixer["scale"], window)
    return mixed.reshape(n, heads * dv) @ w[prefix + "o"].T


def relu_squared_mlp(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str) -> torch.Tensor:
    return (torch.relu(h @ w[prefix + "up"].T) ** 2) @ w[prefix + "down"].T


def layer(x: torch.Tensor, w: Dict[str, torch.Tensor], i: int, cfg: dict) -> torch.Tensor:
    eps, spec, p = cfg["norm"]["eps"], cfg["layers"][i], f"l{i}."
    branches = attention(layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps), w, p + "mix.", spec["mixer"], eps)
    if spec.get("mlp") is not None:
        branches = branches + relu_squared_mlp(layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps), w, p + "mlp.")
    return x + cfg["residual_mult"] * branches


def layer_order(cfg: dict) -> List[tuple]:
    """``(layer, starts a pass)`` for every run of a layer."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    order = [(i, False) for i in range(loop["start"])]
    for _ in range(loop["times"]):
        order += [(i, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return order + [(i, False) for i in range(loop["stop"], n)]


def forward(cfg: dict, weights: Dict[str, torch.Tensor], ids: Sequence[int], streams: Optional[list] = None) -> torch.Tensor:
    """Logits ``[n, vocab]`` of the whole sequence; ``streams`` (a list) receives the stream after every run of a layer."""
    w = {name: t.to(F64) for name, t in weights.items()}
    n = len(ids)
    x0 = w["embed"][torch.tensor(list(ids), dtype=torch.long)] + w["pos"][:n]
    x = x0
    for i, starts_pass in layer_order(cfg):
        if starts_pass:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T
        x = layer(x, w, i, cfg)
        if streams is not None:
            streams.append(x)
    return layer_norm(x, w["final.norm"], w["final.norm.b"], cfg["norm"]["eps"]) @ w["head"].T
