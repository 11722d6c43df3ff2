"""Position encodings.

``LearnedPositions``: a table of position vectors added to the token embedding;
the row for position p is ``p + offset``.  The reference strips the first
``offset`` = 2 rows of OPT's table when converting (scripts/lib/converter_lib.py:271)
and indexes by p (src/csrc/kernel/embedding.cu:25-35); the table stays whole here.
``NoPositions``: nothing is added (the reference passes a null table for rotary
models, src/csrc/model/gpt/gpt.cc:138)."""
from __future__ import annotations

from typing import Dict, List

import torch

from ..weights.loader import TensorSpec
from .base import PositionEncoding


class LearnedPositions(PositionEncoding):
    """params: max_positions (int), offset (int)."""

    def __init__(self, spec, hidden_size, dtype):
        super().__init__(spec, hidden_size, dtype)
        self.max_positions = int(self.param("max_positions"))
        self.offset = int(spec.params.get("offset", 0))
        self.table = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name("weight"), (self.max_positions + self.offset, self.hidden_size),
                           "table")]

    def bind(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors[self.name("weight")]

    def embedding_addend(self, ctx):
        """(table, row index tensor, constant added to the index)."""
        return self.table, ctx.positions, self.offset


class NoPositions(PositionEncoding):
    pass
