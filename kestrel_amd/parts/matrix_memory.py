"""A gated matrix memory: a recurrent mixer with a state of fixed size per request."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import core
from ..ops.linear import linear
from .base import LayerCache, Mixer, register_mixer
from .specs import MatrixMemorySpec, ParamSpec, StateSpec


class MatrixMemory(Mixer):
    """Per head a matrix ``S`` ``[hd, hdv]``, a normaliser ``n`` ``[hd]`` and a running maximum ``m`` of the gates'
    logarithms, all fp32, zero for a new request and carried from token to token in the request's state slot.

    With ``q = W_q h * hd ** -0.5``, ``k = W_k h``, ``v = W_v h`` split into heads, and per head the log gates
    ``li = cap * tanh((W_in h + b_in) / cap)`` and ``lf = logsigmoid(cap * tanh((W_keep h + b_keep) / cap))``:

        m' = max(lf + m, li)
        S' = exp(lf + m - m') S + exp(li - m') k v^T        (n' the same with k alone)
        o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)

    Every head's ``o`` is divided by its root mean square (``eps``), the heads are concatenated, multiplied by the gain
    ``norm.weight`` and by ``sigmoid(W_gate h)``, and go through the output projection.

    One launch projects q | k | v | gate in the activation type; the two gates' pre-activations come from a linear of their
    own with fp32 output (what enters the recurrence stays in 32 bits); one kernel then walks over every row's tokens in
    order (``ops.core.matrix_memory``), whatever the step holds: a prompt, a portion, single tokens. In bf16, steps that
    hold more than single tokens go to a kernel that unrolls the recurrence over chunks of 64 tokens into products on the
    matrix cores, where it covers the head sizes. Rows without a
    request (the padding of a replayed step) write zeros and touch no state."""

    replays_every_step = True
    # Tokens of a step from which the chunks of a row are run at once, in three passes, instead of in turn (a chain of
    # chunks of 46 us each against three launches)
    PASSES_FROM_TOKENS = 192

    def __init__(self, spec: MatrixMemorySpec) -> None:
        super().__init__(spec)
        self.qk_dim = spec.n_heads * spec.head_dim
        self.v_dim = spec.n_heads * spec.value_dim
        self.gated = bool(spec.output_gate)
        self.in_dim = 2 * self.qk_dim + self.v_dim * (2 if self.gated else 1)
        self.in_weight = self.gates_weight = self.gates_bias = self.gain = self.proj_weight = None
        self.dtype: Optional[torch.dtype] = None

    def params(self) -> Dict[str, ParamSpec]:
        spec = self.spec
        out = {"q.weight": ParamSpec((self.qk_dim, spec.dim)), "k.weight": ParamSpec((self.qk_dim, spec.dim)),
               "v.weight": ParamSpec((self.v_dim, spec.dim)), "proj.weight": ParamSpec((spec.dim, self.v_dim)),
               "norm.weight": ParamSpec((self.v_dim,), "vector", "gain"),
               "in.weight": ParamSpec((spec.n_heads, spec.dim)), "in.bias": ParamSpec((spec.n_heads,), "vector", "bias"),
               "keep.weight": ParamSpec((spec.n_heads, spec.dim)), "keep.bias": ParamSpec((spec.n_heads,), "vector", "bias")}
        if self.gated:
            out["gate.weight"] = ParamSpec((self.v_dim, spec.dim))
        return out

    def state_spec(self) -> StateSpec:
        spec = self.spec
        return StateSpec((spec.n_heads * (spec.head_dim * spec.value_dim + spec.head_dim + 1),), "float32")

    def bind(self, tensors, dtype, device) -> None:
        self.dtype = dtype
        names = ["q.weight", "k.weight", "v.weight"] + (["gate.weight"] if self.gated else [])
        self.in_weight = torch.cat([tensors[name].to(device) for name in names], dim=0).contiguous()
        self.gates_weight = torch.cat([tensors["in.weight"].to(device), tensors["keep.weight"].to(device)], dim=0).contiguous()
        self.gates_bias = torch.cat([tensors["in.bias"].to(device=device, dtype=torch.float32),
                                     tensors["keep.bias"].to(device=device, dtype=torch.float32)]).contiguous()
        self.gain = tensors["norm.weight"].to(device=device, dtype=torch.float32).contiguous()
        self.proj_weight = tensors["proj.weight"].to(device).contiguous()

    def read(self, h, batch, cache: LayerCache) -> torch.Tensor:
        """The recurrence over the step's tokens; returns the input of the output projection ``[n, heads hdv]``."""
        spec = self.spec
        n = h.shape[0]
        ws = batch.workspace
        projected = ws.get("memory.in", (n, self.in_dim), self.dtype)
        linear(h, self.in_weight, None, projected)
        pre = ws.get("memory.gates", (n, 2 * spec.n_heads), torch.float32)
        linear(h, self.gates_weight, self.gates_bias, pre)
        out = ws.get("memory.out", (n, self.v_dim), self.dtype)
        if cache.state is None:
            raise RuntimeError("the matrix memory needs its per-request state from the cache manager")
        offsets = (0, self.qk_dim, 2 * self.qk_dim, 2 * self.qk_dim + self.v_dim if self.gated else None)
        scratch = None
        if self.dtype == torch.bfloat16 and not batch.decode_only and n >= self.PASSES_FROM_TOKENS:
            # (sized by the host side of the batch alone: the same for every replay of a captured step)
            from ..ops import fast
            need = fast.matrix_memory_chunks_scratch(n, batch.n_rows, spec.n_heads, spec.head_dim, spec.value_dim)
            if need:
                scratch = ws.get("memory.chunks", (need,), torch.float32)
        core.matrix_memory(projected, offsets, pre, cache.state, batch.cu_q, batch.row_slot, self.gain, out, spec.n_heads,
                           spec.head_dim, spec.value_dim, float(spec.head_dim) ** -0.5, spec.gate_cap, spec.eps,
                           single_tokens=bool(batch.decode_only), chunks=True, scratch=scratch)
        return out

    def output_projection(self):
        return self.proj_weight, None

    def mix(self, h, batch, cache: LayerCache, out, accumulate: bool) -> None:
        """The mixer's output written into (or added to) fp32 ``out``."""
        linear(self.read(h, batch, cache), self.proj_weight, None, out, accumulate=accumulate)

    def forward(self, h, batch, cache: LayerCache, residual) -> None:
        self.mix(h, batch, cache, residual, True)


register_mixer("matrix_memory", MatrixMemory)
