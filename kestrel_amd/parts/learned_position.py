"""Learned position vectors, added to the embedded tokens before the first block."""

from __future__ import annotations

from typing import Dict, Optional

import torch

from ..ops import core
from .base import PositionEncoding, register_position
from .specs import LearnedPositionSpec, ParamSpec


class LearnedPositions(PositionEncoding):
    """``x[t] += table[p_t]`` for a token at place ``p_t`` of its sequence (counted from 0), unscaled, in fp32.
    Inside a mixer it offers no rotation: order then reaches attention through the embeddings alone."""

    replays_every_step = True

    def __init__(self, spec: LearnedPositionSpec) -> None:
        super().__init__(spec)
        self._table: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, ParamSpec]:
        return {"table": ParamSpec((self.spec.max_positions, self.spec.dim))}

    def bind(self, tensors, dtype, device) -> None:
        self._table = tensors["table"].to(device).contiguous()

    def add_to_embeddings(self, x, batch) -> None:
        core.add_table_rows(self._table, batch.positions, x)


register_position("learned", LearnedPositions)
