"""Norms. LayerNorm with gain and offset, its epsilon a parameter (the reference fixes 1e-5 in
code: engine/src/gpt2_gpu.cu:15; formula engine/src/layernorm.c:15-33)."""

from __future__ import annotations

from ..ops import kernels
from ..weights.spec import VECTOR, Normal, TensorSpec
from .base import Norm, register_part


class LayerNorm(Norm):
    takes_pending = True

    def __init__(self, width: int, eps: float):
        self.width, self.eps = width, eps
        self.weight = None
        self.bias = None

    def tensor_specs(self):
        return {
            "weight": TensorSpec((self.width,), VECTOR, Normal(0.05, mean=1.0)),
            "bias": TensorSpec((self.width,), VECTOR, Normal(0.02)),
        }

    def forward(self, x, out_dtype, row_index=None):
        return kernels.layernorm(x, self.weight, self.bias, self.eps, out_dtype=out_dtype, row_index=row_index)

    def forward_into(self, x, out):
        return kernels.layernorm(x, self.weight, self.bias, self.eps, out_dtype=out.dtype, out=out)

    def forward_with_sums(self, hidden, out_dtype, packed=False):
        return kernels.layernorm(hidden, self.weight, self.bias, self.eps, out_dtype=out_dtype, with_sums=True, packed_out=packed)


register_part("norm", "layernorm", LayerNorm)
