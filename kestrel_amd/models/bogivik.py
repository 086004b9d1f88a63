"""Bogivik: a small decoder whose layers mix tokens either by attention with a learned distance bias or by two mixers
side by side, chunked rotary attention and a gated matrix memory.

The design, in this file's notation (``w`` the width, ``eps`` the one epsilon of all norms, ``rms(x) = x / sqrt(mean(x^2) + eps)``):

* ``x = embed[token]``; a layer is ``h = rms(x) * norm1``, ``x <- x + mix(h) + mlp(h)``: one norm, read by both branches; a layer
  whose ``mlp`` is null has the first branch only. Logits are ``head(rms(x) * final.norm)``.
* ``mlp`` (``kind`` ``dense``): ``down(gelu_tanh(gate h) * (up h))``, no biases.
* Layer type ``attention``: ``heads`` query heads over ``kv_heads`` key/value heads, keys of ``dim`` and values of ``vdim``
  channels, no biases, no rotation. All queries of a token are normalised together, ``rms(W_q h) * q.norm`` over the whole
  projection, likewise the keys. The query at place ``p`` is multiplied by ``1 + coef * ln(floor((p + 1) / every) + 1)``
  (``q_temp``). The score is ``scale * (q . k) + rel[bucket(i - j), head]``, the buckets of ``parts.specs.DistanceBuckets``
  with ``rel``'s rows and ``bias_max`` as the far distance; every ``j <= i`` is seen. In every layer that says ``v_mix``,
  but the first of them, the values become ``(1 - vmix) v + vmix v_first`` with the first such layer's values of the same
  token, and that is what is cached. The concatenated heads are multiplied by ``sigmoid(W_g h)`` before ``W_o``.
* Layer type ``parallel``: ``0.5 * (rms(left(h)) * left.out + rms(right(h)) * right.out)`` over the width.
  ``left``: attention with biases on q, k, v and o, every query and key head normalised by itself with one gain of a
  head's size (``q.norm``, ``k.norm``), then rotated on the first ``rot.dims`` channels with channels ``2i`` and ``2i + 1`` as a pair
  and the frequencies ``rot.base ** (-2i / dims)`` rescaled by wavelength (``rot.scaling``); a query reads the keys ``j <= i`` of
  its own chunk of ``mask.size`` places; the same output gate.
  ``right``: the gated matrix memory of ``parts/matrix_memory.py`` with ``gate_cap``.

Every size and constant above that is not a literal comes from ``config.json`` or from a tensor's shape. Tensor names: ``embed``,
``l<i>.norm1``, ``l<i>.mix.{q,k,v,g,o}``, ``l<i>.mix.{q,k}.norm``, ``l<i>.mix.rel``, ``l<i>.mix.vmix``, ``l<i>.mix.left.*`` (with ``.b``
for biases), ``l<i>.mix.right.{q,k,v,g,o,norm,i,i.b,f,f.b}``, ``l<i>.mix.{left,right}.out``, ``l<i>.mlp.{gate,up,down}``,
``final.norm``, ``head``.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.registry import ModelSpec, register
from ..parts.specs import (AttentionSpec, BranchesSpec, DistanceBuckets, GatedFeedForwardSpec, LayerSpec, MatrixMemorySpec,
                           ModelPlan, NormSpec, PositionSpec, QKNorm, QueryGrowth, ScheduleEntry, ValueBlend,
                           WavelengthScaling)

NAME = "bogivik"
MLP_ACTIVATION = "gelu_tanh"
BRANCH_WEIGHTS = (0.5, 0.5)            # the parallel mixer is half the sum of its two normalised branches
VALUE_BLEND_NAME = "first_values"
# The design has no longest sequence of its own (no table depends on one). ``config.json`` may name a bound
# (``max_positions``); without one this stands, and the engine's ``max_seq_len`` narrows it (captured steps carry
# block tables of that many positions).
DEFAULT_MAX_POSITIONS = 1 << 17


def _positive_int(where: str, value) -> int:
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ValueError(f"config.json: {where} must be a positive integer, got {value!r}")
    return value


def _number(where: str, value) -> float:
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ValueError(f"config.json: {where} must be a number, got {value!r}")
    return float(value)


def _object(where: str, value, keys=()) -> dict:
    if not isinstance(value, dict):
        raise ValueError(f"config.json: {where} must be an object")
    for key in keys:
        if key not in value:
            raise ValueError(f"config.json: {where}.{key} missing")
    return value


@dataclass(frozen=True)
class BogivikAttention:
    """Sizes of an attention mixer; the options a kind of layer does not have are ``None``."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    # layer type ``attention``
    bias_max: Optional[float] = None
    buckets: Optional[int] = None                      # rows of ``rel``; None: as the weights file has them
    q_temp: Optional[Tuple[float, int]] = None         # (coef, every)
    v_mix: bool = False
    # the left branch of layer type ``parallel``
    chunk: Optional[int] = None
    rot_dims: int = 0
    rot_base: float = 0.0
    rot_scaling: Optional[Tuple[float, float, float, float]] = None     # (factor, low, high, original)

    @classmethod
    def read(cls, where: str, m: dict, left: bool) -> "BogivikAttention":
        _object(where, m, ("heads", "kv_heads", "dim", "vdim", "scale"))
        heads, kv_heads = _positive_int(f"{where}.heads", m["heads"]), _positive_int(f"{where}.kv_heads", m["kv_heads"])
        if heads % kv_heads:
            raise ValueError(f"config.json: {where}: {heads} heads are no multiple of {kv_heads} kv_heads")
        common = dict(heads=heads, kv_heads=kv_heads, dim=_positive_int(f"{where}.dim", m["dim"]),
                      vdim=_positive_int(f"{where}.vdim", m["vdim"]), scale=_number(f"{where}.scale", m["scale"]))
        if left:
            mask = _object(f"{where}.mask", m.get("mask"), ("size",))
            rot = _object(f"{where}.rot", m.get("rot"), ("base", "dims"))
            dims = _positive_int(f"{where}.rot.dims", rot["dims"])
            if dims % 2 or dims > common["dim"]:
                raise ValueError(f"config.json: {where}.rot.dims must be even and at most dim, got {dims}")
            scaling = rot.get("scaling")
            if scaling is not None:
                _object(f"{where}.rot.scaling", scaling, ("factor", "low", "high", "original"))
                scaling = tuple(_number(f"{where}.rot.scaling.{k}", scaling[k]) for k in ("factor", "low", "high", "original"))
            return cls(**common, chunk=_positive_int(f"{where}.mask.size", mask["size"]), rot_dims=dims,
                       rot_base=_number(f"{where}.rot.base", rot["base"]), rot_scaling=scaling)
        if "bias_max" not in m:
            raise ValueError(f"config.json: {where}.bias_max missing")
        temp = m.get("q_temp")
        if temp is not None:
            _object(f"{where}.q_temp", temp, ("coef", "every"))
            temp = (_number(f"{where}.q_temp.coef", temp["coef"]), _positive_int(f"{where}.q_temp.every", temp["every"]))
        buckets = m.get("buckets")       # (not a key of the design: only the writer of random weights needs the number)
        if buckets is not None:
            buckets = _positive_int(f"{where}.buckets", buckets)
        return cls(**common, bias_max=_number(f"{where}.bias_max", m["bias_max"]), buckets=buckets, q_temp=temp,
                   v_mix=bool(m.get("v_mix", False)))

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.chunk is not None:
            out["mask"] = {"size": self.chunk}
            out["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_scaling is not None:
                out["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), self.rot_scaling))
        else:
            out["bias_max"] = self.bias_max
            out["v_mix"] = self.v_mix
            if self.buckets is not None:
                out["buckets"] = self.buckets
            if self.q_temp is not None:
                out["q_temp"] = {"coef": self.q_temp[0], "every": self.q_temp[1]}
        return out


@dataclass(frozen=True)
class BogivikMemory:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def read(cls, where: str, m: dict) -> "BogivikMemory":
        _object(where, m, ("heads", "dim", "vdim", "gate_cap"))
        cap = _number(f"{where}.gate_cap", m["gate_cap"])
        if not cap > 0:
            raise ValueError(f"config.json: {where}.gate_cap must be positive")
        return cls(_positive_int(f"{where}.heads", m["heads"]), _positive_int(f"{where}.dim", m["dim"]),
                   _positive_int(f"{where}.vdim", m["vdim"]), cap)

    def to_dict(self) -> Dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class BogivikLayer:
    kind: str                                  # "attention" or "parallel"
    attention: BogivikAttention                # the mixer of an attention layer, the left branch of a parallel one
    memory: Optional[BogivikMemory]            # the right branch of a parallel layer
    ff: Optional[int]                          # hidden size of the feed-forward; None: the layer has none


@dataclass(frozen=True)
class BogivikConfig:
    vocab: int
    width: int
    eps: float
    max_positions: int
    layers: Tuple[BogivikLayer, ...]
    raw: Any = None

    @classmethod
    def from_dict(cls, config: Dict[str, Any]) -> "BogivikConfig":
        for key in ("layers", "vocab", "width", "norm"):
            if key not in config:
                raise ValueError(f"config.json: key {key!r} missing")
        eps = _number("norm.eps", _object("norm", config["norm"], ("eps",))["eps"])
        if not eps >= 0:
            raise ValueError("config.json: norm.eps must not be negative")
        listed = config["layers"]
        if not isinstance(listed, list) or not listed:
            raise ValueError("config.json: 'layers' must be a list of layers")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            _object(where, entry, ("type", "mixer"))
            kind = entry["type"]
            mixer = _object(f"{where}.mixer", entry["mixer"])
            if kind == "attention":
                attention, memory = BogivikAttention.read(f"{where}.mixer", mixer, left=False), None
            elif kind == "parallel":
                _object(f"{where}.mixer", mixer, ("left", "right"))
                attention = BogivikAttention.read(f"{where}.mixer.left", mixer["left"], left=True)
                memory = BogivikMemory.read(f"{where}.mixer.right", mixer["right"])
            else:
                raise ValueError(f"config.json: {where}.type is {kind!r}; this design has the mixers 'attention' and 'parallel'")
            mlp = entry.get("mlp")
            ff = None
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ValueError(f"config.json: {where}.mlp must be null or an object of kind 'dense'")
                ff = _positive_int(f"{where}.mlp.ff", mlp.get("ff"))
            layers.append(BogivikLayer(kind, attention, memory, ff))
        blending = [layer.attention for layer in layers if layer.kind == "attention" and layer.attention.v_mix]
        if any((a.kv_heads, a.vdim) != (blending[0].kv_heads, blending[0].vdim) for a in blending):
            raise ValueError("config.json: layers that blend their values must have values of one shape")
        positions = config.get("max_positions", DEFAULT_MAX_POSITIONS)
        return cls(vocab=_positive_int("vocab", config["vocab"]), width=_positive_int("width", config["width"]), eps=eps,
                   max_positions=_positive_int("max_positions", positions), layers=tuple(layers), raw=config)

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for layer in self.layers:
            mixer = layer.attention.to_dict() if layer.kind == "attention" else \
                {"left": layer.attention.to_dict(), "right": layer.memory.to_dict()}
            layers.append({"type": layer.kind, "mixer": mixer, "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}})
        out = {"architecture": "Bogivik", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps}, "layers": layers}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out


def _attention_names(prefix: str, local: str, biases: bool) -> Dict[str, str]:
    """Tensor names of an attention mixer whose local names start with ``local`` and whose tensors with ``prefix``."""
    names = {f"{local}q.weight": prefix + "q", f"{local}k.weight": prefix + "k", f"{local}v.weight": prefix + "v",
             f"{local}gate.weight": prefix + "g", f"{local}proj.weight": prefix + "o",
             f"{local}q_norm.weight": prefix + "q.norm", f"{local}k_norm.weight": prefix + "k.norm"}
    if biases:
        names.update({f"{local}q.bias": prefix + "q.b", f"{local}k.bias": prefix + "k.b", f"{local}v.bias": prefix + "v.b",
                      f"{local}proj.bias": prefix + "o.b"})
    return names


def build_plan(cfg: BogivikConfig) -> ModelPlan:
    layers = []
    ignored = []
    first_blend_seen = False
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        a = layer.attention
        names = {"norm.weight": p + "norm1"}
        if layer.kind == "attention":
            blend = None
            if a.v_mix:
                blend = ValueBlend("blend" if first_blend_seen else "source", VALUE_BLEND_NAME)
                first_blend_seen = True
                names["mixer.vmix"] = p + "mix.vmix"
            else:
                ignored.append(p + "mix.vmix")
            mixer = AttentionSpec(
                "attention", cfg.width, a.heads, a.kv_heads, a.dim, PositionSpec("none"), bias=False, scale=a.scale,
                value_dim=a.vdim, split_projections=True, qk_norm=QKNorm("projection", cfg.eps),
                query_growth=QueryGrowth(*a.q_temp) if a.q_temp is not None else None,
                distance_buckets=DistanceBuckets(a.buckets, a.bias_max),
                value_blend=blend, output_gate=True)
            names.update(_attention_names(p + "mix.", "mixer.", biases=False))
            names["mixer.rel"] = p + "mix.rel"
        else:
            m = layer.memory
            rotation = PositionSpec("rotary", rotary_dim=a.rot_dims, theta=a.rot_base, pairing="interleaved",
                                    scaling=WavelengthScaling(*a.rot_scaling) if a.rot_scaling is not None else None)
            left = AttentionSpec("attention", cfg.width, a.heads, a.kv_heads, a.dim, rotation, bias=True, scale=a.scale,
                                 value_dim=a.vdim, split_projections=True, qk_norm=QKNorm("head", cfg.eps), chunk=a.chunk,
                                 output_gate=True)
            right = MatrixMemorySpec("matrix_memory", cfg.width, m.heads, m.dim, m.vdim, m.gate_cap, cfg.eps, output_gate=True)
            mixer = BranchesSpec("branches", cfg.width, (left, right), BRANCH_WEIGHTS, cfg.eps)
            names.update(_attention_names(p + "mix.left.", "mixer.0.", biases=True))
            r = p + "mix.right."
            names.update({"mixer.1.q.weight": r + "q", "mixer.1.k.weight": r + "k", "mixer.1.v.weight": r + "v",
                          "mixer.1.gate.weight": r + "g", "mixer.1.proj.weight": r + "o", "mixer.1.norm.weight": r + "norm",
                          "mixer.1.in.weight": r + "i", "mixer.1.in.bias": r + "i.b", "mixer.1.keep.weight": r + "f",
                          "mixer.1.keep.bias": r + "f.b", "mixer.out0.weight": p + "mix.left.out",
                          "mixer.out1.weight": p + "mix.right.out"})
        feed_forward = None
        if layer.ff is not None:
            feed_forward = GatedFeedForwardSpec("gated_dense", cfg.width, layer.ff, MLP_ACTIVATION, bias=False)
            names.update({"feed_forward.gate.weight": p + "mlp.gate", "feed_forward.up.weight": p + "mlp.up",
                          "feed_forward.down.weight": p + "mlp.down"})
        layers.append(LayerSpec(arrangement="parallel", norm=NormSpec("rmsnorm", cfg.width, cfg.eps, bias=False), mixer=mixer,
                                feed_forward=feed_forward, names=names))
    return ModelPlan(
        architecture=NAME, vocab_size=cfg.vocab, dim=cfg.width, max_positions=cfg.max_positions, layers=tuple(layers),
        schedule=tuple(ScheduleEntry(i) for i in range(len(layers))),
        final_norm=NormSpec("rmsnorm", cfg.width, cfg.eps, bias=False), head_bias=False, tied_head=False,
        names={"embedding": "embed", "final_norm.weight": "final.norm", "head.weight": "head"},
        ignored_prefixes=tuple(ignored),
    )


def _claims(config: Dict[str, Any]) -> bool:
    layers = config.get("layers")
    return isinstance(layers, list) and bool(layers) and "residual_mult" not in config and "width" in config and \
        all(isinstance(e, dict) and e.get("type") in ("attention", "parallel") and "mixer" in e for e in layers) and \
        any(e.get("type") == "parallel" or "bias_max" in (e.get("mixer") or {}) for e in layers)


register(ModelSpec(
    name=NAME,
    read_config=BogivikConfig.from_dict,
    build_plan=build_plan,
    aliases=("Bogivik",),
    claims=_claims,
    filename="model.safetensors",
))
