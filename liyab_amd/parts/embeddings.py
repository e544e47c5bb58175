"""Token embedding and position encodings that act on the residual stream."""

from __future__ import annotations

from typing import Optional

import torch

from ..kernels import ops
from .base import StepContext
from .registry import register_embedding, register_position


class TokenEmbedding:
    """x[t] = scale * table[id_t] (the reference's embed, src/core/transformer.cpp:5495-5512).
    A residual position table may be folded into the same pass."""

    takes_padding_rows = True  # (they carry token 0)

    def __init__(self, spec, store, dtype: torch.dtype):
        self.vocab_size, self.width, self.scale = spec.vocab_size, spec.width, float(spec.scale)
        self.table = store.fetch(spec.tensors["table"], (self.vocab_size, self.width), "table")

    def forward(self, ctx: StepContext, x: torch.Tensor, position_table: Optional[torch.Tensor] = None) -> None:
        ops.embed(x, self.table, ctx.token_ids, self.scale, pos_table=position_table,
                  positions=ctx.positions if position_table is not None else None, last_tokens=ctx.last_tokens)


class LearnedPositions:
    """x[t] += table[pos_t] (the reference's add_positions, src/core/transformer.cpp:2791-2808).
    The only position encoding that caps the context at its table's rows (:819-823)."""

    where = "residual"
    takes_padding_rows = True  # (they sit at position 0)

    def __init__(self, spec, store, dtype: torch.dtype):
        self.max_positions, self.width = spec.max_positions, spec.width
        self.table = store.fetch(spec.tensors["table"], (self.max_positions, self.width), "table")

    def fused_table(self) -> Optional[torch.Tensor]:
        """The table, when the embedding kernel may add it in its own pass."""
        return self.table

    def add(self, ctx: StepContext, x: torch.Tensor) -> None:
        ops.add_rows_(x, self.table, ctx.positions)


register_embedding("token_embedding", TokenEmbedding)
register_position("learned_positions", LearnedPositions)
