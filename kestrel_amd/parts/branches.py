"""Mixers side by side: several mixers read the same input, their normalised outputs are summed with weights."""

from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import core
from .base import LayerCache, Mixer, build_part, register_mixer
from .specs import BranchesSpec, ParamSpec


class Branches(Mixer):
    """``sum_i weights[i] * rms(branch_i(h)) * gain_i``: every branch is a mixer of any registered kind, built from its
    own specification; its output ``[n, dim]`` is divided by its root mean square over the model width (``eps``) and
    multiplied by a gain of its own (tensor ``out<i>.weight``) before the weighted sum enters the stream.

    The tensors of branch ``i`` are named ``<i>.<local name>``. What the branches keep is the layer's: at most one of
    them may keep keys and values per token and at most one a state per request (a layer has one cache group and one
    state tensor); each gets the layer's ``LayerCache`` and takes from it what is its own."""

    def __init__(self, spec: BranchesSpec) -> None:
        super().__init__(spec)
        if not spec.branches or len(spec.branches) != len(spec.weights) or len(spec.branches) > 2:
            raise ValueError("branches: one or two mixers, and a weight for each")
        self.branches: List[Mixer] = [build_part("mixer", b) for b in spec.branches]
        if sum(b.cache_spec() is not None for b in self.branches) > 1 or sum(b.state_spec() is not None for b in self.branches) > 1:
            raise ValueError("branches: at most one branch may keep a cache per token and at most one a state per request")
        self.gains: List[Optional[torch.Tensor]] = [None] * len(self.branches)
        self.dtype: Optional[torch.dtype] = None

    @property
    def replays_every_step(self) -> bool:
        return all(bool(getattr(b, "replays_every_step", False)) for b in self.branches)

    @property
    def position(self):
        """(the runner asks a mixer's position encoding how many numbers it takes per token)"""
        return next((getattr(b, "position", None) for b in self.branches if getattr(b, "position", None) is not None), None)

    def params(self) -> Dict[str, ParamSpec]:
        out = {}
        for i, branch in enumerate(self.branches):
            out.update({f"{i}.{name}": pspec for name, pspec in branch.params().items()})
            out[f"out{i}.weight"] = ParamSpec((self.spec.dim,), "vector", "gain")
        return out

    def bind(self, tensors, dtype, device) -> None:
        self.dtype = dtype
        for i, branch in enumerate(self.branches):
            branch.bind({name: tensors[f"{i}.{name}"] for name in branch.params()}, dtype, device)
            self.gains[i] = tensors[f"out{i}.weight"].to(device=device, dtype=torch.float32).contiguous()

    def cache_spec(self):
        return next((b.cache_spec() for b in self.branches if b.cache_spec() is not None), None)

    def state_spec(self):
        return next((b.state_spec() for b in self.branches if b.state_spec() is not None), None)

    def query_tile(self):
        return next((b.query_tile() for b in self.branches if b.query_tile()), None)

    def forward(self, h, batch, cache: LayerCache, residual) -> None:
        n = h.shape[0]
        outs = []
        for i, branch in enumerate(self.branches):
            out = batch.workspace.get(f"branches.out{i}", (n, self.spec.dim), torch.float32)
            mix = getattr(branch, "mix", None)
            if callable(mix):
                mix(h, batch, cache, out, False)
            else:
                out.zero_()              # (a fill kernel: a mixer that only knows how to add)
                branch.forward(h, batch, cache, out)
            outs.append(out)
        second = len(outs) > 1
        core.branches_sum(residual, outs[0], self.gains[0], self.spec.weights[0], outs[1] if second else None,
                          self.gains[1] if second else None, self.spec.weights[1] if second else 0.0, self.spec.eps)


register_mixer("branches", Branches)
