"""Positions that enter the model as a learned row added to the embedded token."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..kernels import ops, profile
from ..weights.spec import INIT_NORMAL, TABLE, TensorSpec
from .base import PositionEncoding, register_part


class LearnedPositions(PositionEncoding):
    """``x[t] = x[t] * input_scale + table[position of t]``: the table's row is added as it is;
    ``input_scale`` is what the embedded rows are multiplied by first (an embedding's scale), so
    that scale and sum are one pass over the rows.  Positions count from 0 in every request and
    must stay below ``max_positions``: the step function refuses a step that would go past
    (``Model.position_limit``); a batch's ``max_position`` may be a bound only (a captured decode
    graph's), so it is no test here."""

    def __init__(self, name: str, max_positions: int, width: int, input_scale: float = 1.0):
        self.name, self.max_positions, self.width = name, int(max_positions), width
        self.input_scale = float(input_scale)
        self.table: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name, (self.max_positions, self.width), TABLE, INIT_NORMAL)]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors[self.name].contiguous()

    def on_embedding(self, x: torch.Tensor, batch) -> None:
        with profile.scope("embd"):
            ops.scale_add_positions(x, self.input_scale, self.table, batch.row_pos)


register_part("position_encoding", "learned", LearnedPositions)
