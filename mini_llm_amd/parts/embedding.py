"""The token table, read at the bottom of the model (gather) and, tied, at the top (head)."""

from __future__ import annotations

from ..ops import kernels
from ..weights.spec import TABLE, Normal, TensorSpec
from .base import Part, PositionEncoding


class TokenEmbedding(Part):
    def __init__(self, vocab_size: int, width: int):
        self.vocab_size, self.width = vocab_size, width
        self.weight = None

    def tensor_specs(self):
        return {"weight": TensorSpec((self.vocab_size, self.width), TABLE, Normal(0.02))}

    def forward(self, tokens, positions, position_encoding: PositionEncoding | None, token_sources=None, token_slots=None):
        """[rows, width] float32: token rows, with the position rows added when the encoding
        is one that enters at the embedding (a table ``weight`` [positions, width]); an encoding
        of stage "mixer", or none, leaves the token rows as they are. ``token_sources`` /
        ``token_slots``: rows whose token is still on the device, in the slot the sampler left it
        in (kernels.embed)."""
        table = position_encoding.weight if position_encoding is not None and position_encoding.stage == "embedding" else None
        return kernels.embed(tokens, positions, self.weight, table, token_sources=token_sources, token_slots=token_slots)


class TiedHead(Part):
    """logits = x . wte^T, no bias, no tensor of its own (engine/src/gpt2.c:244-256)."""

    def __init__(self, embedding: TokenEmbedding):
        self.embedding = embedding

    def forward(self, x):
        import torch

        return kernels.linear(x, self.embedding.weight, out_dtype=torch.float32)

    def forward_best(self, x):
        """For a step that decodes greedily: instead of the logits, per row the best (logit, token) of each of a few
        hundred disjoint parts of the vocabulary (kernels.linear_best), among which ``kernels.choose`` finds the row's
        argmax; None where that kernel does not take the sizes (the caller then takes the logits). A head without this
        method is asked for its logits."""
        if not kernels.best_per_row(x.shape[0], self.embedding.weight, x.dtype):
            return None
        return kernels.linear_best(x, self.embedding.weight)
