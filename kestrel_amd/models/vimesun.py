"""Vimesun: a small decoder whose order comes from learned position vectors and from a distance bias
inside attention, with a stretch of its layers run several times.

The design, in this file's notation (``w`` the width, ``eps`` the one epsilon of all norms):

* ``x0 = embed[token] + pos[p]`` for a token at place ``p`` of its sequence.
* The layers ``start .. stop - 1`` of ``loop`` run ``times`` times in a row with the same weights and a cache
  of their own each time; every such pass begins with ``x <- loop.in [x; x0]`` (``[w, 2 w]``).
* A layer: ``x <- x + residual_mult * (mix(LN1(x)) + mlp(LN2(x)))``, two LayerNorms (gain and shift) of the same
  ``x``; a layer whose ``mlp`` is null has the first branch only.
* ``mix``: attention without biases and without a rotation. ``heads`` query heads share ``kv_heads`` key/value
  heads; queries and keys have ``dim`` channels a head, values ``vdim``. Queries and keys are divided head by head
  by ``sqrt(mean(square) + eps)``. The score of a query at ``i`` against the key at ``j`` is
  ``scale * (q . k) - 2 ** (-8 (h + 1) / heads) * (i - j)`` for head ``h``; a query sees ``0 <= i - j < mask.size``;
  the softmax's denominator has one more term of score 0 and no value.
* ``mlp`` (``kind`` ``dense``): ``down(relu(up(h)) ** 2)``, no biases.
* Logits: ``head(LN(x))`` with the LayerNorm ``final.norm``; the head is not tied and has no bias.

Every size and constant above that is not a literal comes from ``config.json`` or from a tensor's shape.
Tensor names: ``embed``, ``pos``, ``loop.in``, ``l<i>.norm1`` (gain) and ``l<i>.norm1.b`` (shift), likewise ``norm2``,
``l<i>.mix.{q,k,v,o}``, ``l<i>.mlp.{up,down}``, ``final.norm``, ``final.norm.b``, ``head``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.registry import ModelSpec, register
from ..parts.specs import (AttentionSpec, ConcatLinearSpec, DenseFeedForwardSpec, DistanceSlopes, LayerSpec,
                           LearnedPositionSpec, ModelPlan, NormSpec, PositionSpec, ScheduleEntry)

NAME = "vimesun"
SLOPE_EXPONENT = 8.0           # slope of head h of H: 2 ** (-8 (h + 1) / H)
SINK_SCORE = 0.0               # the score of the softmax's valueless term
MLP_ACTIVATION = "relu_squared"


def _positive_int(where: str, value) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ValueError(f"config.json: {where} must be a positive integer, got {value!r}")
    return value


def _number(where: str, value) -> float:
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ValueError(f"config.json: {where} must be a number, got {value!r}")
    return float(value)


@dataclass(frozen=True)
class VimesunMixer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]


@dataclass(frozen=True)
class VimesunLayer:
    mixer: VimesunMixer
    ff: Optional[int]              # hidden size of the dense feed-forward; None: the layer has none


@dataclass(frozen=True)
class VimesunConfig:
    vocab: int
    width: int
    max_positions: int
    eps: float
    residual_mult: float
    layers: Tuple[VimesunLayer, ...]
    loop_start: int
    loop_stop: int
    loop_times: int                # 0: no stretch of layers is repeated and there is no ``loop.in``
    raw: Any = None

    @classmethod
    def from_dict(cls, config: Dict[str, Any]) -> "VimesunConfig":
        for key in ("layers", "vocab", "width", "max_positions", "norm", "residual_mult"):
            if key not in config:
                raise ValueError(f"config.json: key {key!r} missing")
        norm = config["norm"]
        if not isinstance(norm, dict) or "eps" not in norm:
            raise ValueError("config.json: 'norm' must be an object with 'eps'")
        eps = _number("norm.eps", norm["eps"])
        if not eps >= 0:
            raise ValueError("config.json: norm.eps must not be negative")
        listed = config["layers"]
        if not isinstance(listed, list) or not listed:
            raise ValueError("config.json: 'layers' must be a list of layers")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            if not isinstance(entry, dict):
                raise ValueError(f"config.json: {where} must be an object")
            if entry.get("type") != "attention":
                raise ValueError(f"config.json: {where}.type is {entry.get('type')!r}; this design has the mixer 'attention'")
            m = entry.get("mixer")
            if not isinstance(m, dict):
                raise ValueError(f"config.json: {where}.mixer must be an object")
            for key in ("heads", "kv_heads", "dim", "vdim", "scale"):
                if key not in m:
                    raise ValueError(f"config.json: {where}.mixer.{key} missing")
            heads, kv_heads = _positive_int(f"{where}.mixer.heads", m["heads"]), _positive_int(f"{where}.mixer.kv_heads", m["kv_heads"])
            if heads % kv_heads:
                raise ValueError(f"config.json: {where}.mixer: {heads} heads are no multiple of {kv_heads} kv_heads")
            mask = m.get("mask")
            window = None
            if mask is not None:
                if not isinstance(mask, dict) or "size" not in mask:
                    raise ValueError(f"config.json: {where}.mixer.mask must be an object with 'size'")
                window = _positive_int(f"{where}.mixer.mask.size", mask["size"])
            mixer = VimesunMixer(heads, kv_heads, _positive_int(f"{where}.mixer.dim", m["dim"]),
                                 _positive_int(f"{where}.mixer.vdim", m["vdim"]), _number(f"{where}.mixer.scale", m["scale"]), window)
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ValueError(f"config.json: {where}.mlp must be null or an object of kind 'dense'")
                ff = _positive_int(f"{where}.mlp.ff", mlp.get("ff"))
            layers.append(VimesunLayer(mixer, ff))
        loop = config.get("loop")
        start = stop = times = 0
        if loop is not None:
            if not isinstance(loop, dict) or any(key not in loop for key in ("start", "stop", "times")):
                raise ValueError("config.json: 'loop' must be an object with 'start', 'stop' and 'times'")
            start, stop, times = (loop[key] for key in ("start", "stop", "times"))
            for key, value in (("start", start), ("stop", stop), ("times", times)):
                if isinstance(value, bool) or not isinstance(value, int) or value < 0:
                    raise ValueError(f"config.json: loop.{key} must be an integer that is not negative, got {value!r}")
            if not start <= stop <= len(layers):
                raise ValueError(f"config.json: loop {start} .. {stop} does not lie within the {len(layers)} layers")
        return cls(vocab=_positive_int("vocab", config["vocab"]), width=_positive_int("width", config["width"]),
                   max_positions=_positive_int("max_positions", config["max_positions"]), eps=eps,
                   residual_mult=_number("residual_mult", config["residual_mult"]), layers=tuple(layers),
                   loop_start=start, loop_stop=stop, loop_times=times, raw=config)

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for layer in self.layers:
            m = layer.mixer
            mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
            if m.window is not None:
                mixer["mask"] = {"size": m.window}
            layers.append({"type": "attention", "mixer": mixer,
                           "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}})
        out = {"architecture": "Vimesun", "vocab": self.vocab, "width": self.width, "max_positions": self.max_positions,
               "norm": {"eps": self.eps}, "residual_mult": self.residual_mult, "layers": layers}
        if self.loop_times or self.loop_stop > self.loop_start:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        return out


def build_plan(cfg: VimesunConfig) -> ModelPlan:
    no_position = PositionSpec("none")
    layers = []
    ignored = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        m = layer.mixer
        names = {"norm.weight": p + "norm1", "norm.bias": p + "norm1.b",
                 "mixer.q.weight": p + "mix.q", "mixer.k.weight": p + "mix.k", "mixer.v.weight": p + "mix.v",
                 "mixer.proj.weight": p + "mix.o"}
        if layer.ff is not None:
            names.update({"norm2.weight": p + "norm2", "norm2.bias": p + "norm2.b",
                          "feed_forward.fc1.weight": p + "mlp.up", "feed_forward.fc2.weight": p + "mlp.down"})
        else:
            ignored.append(p + "norm2")        # (a layer without a feed-forward has no use for its second norm)
        layers.append(LayerSpec(
            arrangement="parallel_two_norms",
            norm=NormSpec("layernorm", cfg.width, cfg.eps, bias=True),
            norm2=NormSpec("layernorm", cfg.width, cfg.eps, bias=True) if layer.ff is not None else None,
            mixer=AttentionSpec("attention", cfg.width, m.heads, m.kv_heads, m.dim, no_position, bias=False, scale=m.scale,
                                window=m.window, value_dim=m.vdim, split_projections=True, qk_unit_norm_eps=cfg.eps,
                                distance_slopes=DistanceSlopes(SLOPE_EXPONENT), sink=SINK_SCORE),
            feed_forward=DenseFeedForwardSpec("dense", cfg.width, layer.ff, MLP_ACTIVATION, bias=False)
            if layer.ff is not None else None,
            names=names, residual_scale=cfg.residual_mult,
        ))
    schedule = [ScheduleEntry(i) for i in range(cfg.loop_start)]
    for _ in range(cfg.loop_times):
        # every pass keeps a cache of its own and begins at the junction
        schedule += [ScheduleEntry(i, before="loop_in" if i == cfg.loop_start else None)
                     for i in range(cfg.loop_start, cfg.loop_stop)]
    schedule += [ScheduleEntry(i) for i in range(cfg.loop_stop, len(cfg.layers))]
    loops = cfg.loop_times > 0 and cfg.loop_stop > cfg.loop_start
    names = {"embedding": "embed", "position.table": "pos", "final_norm.weight": "final.norm",
             "final_norm.bias": "final.norm.b", "head.weight": "head"}
    if loops:
        names["junction.loop_in.weight"] = "loop.in"
    else:
        ignored.append("loop.in")
    return ModelPlan(
        architecture=NAME, vocab_size=cfg.vocab, dim=cfg.width, max_positions=cfg.max_positions,
        layers=tuple(layers), schedule=tuple(schedule),
        final_norm=NormSpec("layernorm", cfg.width, cfg.eps, bias=True), head_bias=False, tied_head=False, names=names,
        position=LearnedPositionSpec("learned", cfg.width, cfg.max_positions),
        junctions={"loop_in": ConcatLinearSpec("concat_linear", cfg.width)} if loops else {},
        ignored_prefixes=tuple(ignored),
    )


def _claims(config: Dict[str, Any]) -> bool:
    layers = config.get("layers")
    return isinstance(layers, list) and bool(layers) and all(isinstance(e, dict) and "mixer" in e and "type" in e for e in layers) \
        and "residual_mult" in config and "width" in config


register(ModelSpec(
    name=NAME,
    read_config=VimesunConfig.from_dict,
    build_plan=build_plan,
    aliases=("Vimesun",),
    claims=_claims,
    filename="model.safetensors",
))
