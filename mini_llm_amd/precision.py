"""The two precisions a model runs in.

``float32``: every tensor and every product in true 32-bit. ``bfloat16``: matrices, tables,
the activations between kernels and the cache pages in bfloat16; sums, norms, softmax, the
residual stream and the logits in 32-bit, and vectors (biases, norm gains) kept in 32-bit."""

from __future__ import annotations

from dataclasses import dataclass

import torch

_ALIASES = {
    "float32": "float32", "fp32": "float32", "f32": "float32",
    "bfloat16": "bfloat16", "bf16": "bfloat16",
}


@dataclass(frozen=True)
class Precision:
    name: str

    @staticmethod
    def from_name(name) -> "Precision":
        if isinstance(name, Precision):
            return name
        if isinstance(name, torch.dtype):
            name = str(name).replace("torch.", "")
        key = _ALIASES.get(str(name).lower())
        if key is None:
            raise ValueError(f"unknown dtype {name!r}: use float32 or bfloat16")
        return Precision(key)

    @property
    def compute(self) -> torch.dtype:
        """Element type of matrices, tables, activations between kernels and cache pages."""
        return torch.float32 if self.name == "float32" else torch.bfloat16

    # These do not depend on the precision; they are named so that no part hard-codes them.
    residual = torch.float32
    vector = torch.float32
    logits = torch.float32
