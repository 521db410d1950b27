"""Position encodings. GPT-2 has learned absolute positions: a table row per position, added to
the token row at the embedding (engine/src/embedding.c:9-16)."""

from __future__ import annotations

from ..weights.spec import TABLE, Normal, TensorSpec
from .base import PositionEncoding, register_part


class LearnedPositions(PositionEncoding):
    stage = "embedding"

    def __init__(self, n_positions: int, width: int):
        self.n_positions, self.width = n_positions, width
        self.weight = None

    def tensor_specs(self):
        return {"weight": TensorSpec((self.n_positions, self.width), TABLE, Normal(0.02))}

    def max_positions(self) -> int:
        return self.n_positions


register_part("position_encoding", "learned", LearnedPositions)
