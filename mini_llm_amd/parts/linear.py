"""A linear map y = x W + b as a part: weight stored [in, out] (GPT-2's Conv1D) or [out, in],
kept [out, in] for the matrix kernels, with the epilogue (activation, residual sum) fused."""

from __future__ import annotations

from ..ops import kernels
from ..weights.spec import MATRIX, VECTOR, Normal, TensorSpec
from .base import Part


class Linear(Part):
    def __init__(self, in_features: int, out_features: int, *, bias: bool = True, stored_in_out: bool = True,
                 weight_std: float = 0.02, bias_std: float = 0.01):
        self.in_features, self.out_features = in_features, out_features
        self.has_bias, self.stored_in_out = bias, stored_in_out
        self.weight_std, self.bias_std = weight_std, bias_std
        self.weight = None
        self.bias = None
        self._split_blocks = {}
        self._accepts_packed = {}

    def tensor_specs(self):
        shape = (self.in_features, self.out_features) if self.stored_in_out else (self.out_features, self.in_features)
        specs = {"weight": TensorSpec(shape, MATRIX, Normal(self.weight_std), keep_transposed=self.stored_in_out)}
        if self.has_bias:
            specs["bias"] = TensorSpec((self.out_features,), VECTOR, Normal(self.bias_std))
        return specs

    def forward(self, x, activation=None, residual=None, out_dtype=None, packed_out=False):
        return kernels.linear(x, self.weight, self.bias, activation=activation, residual=residual, out_dtype=out_dtype, packed_out=packed_out)

    def accepts_packed_rows(self, rows: int, dtype, pending: bool = False) -> bool:
        """Whether ``forward`` (or, with ``pending``, ``forward_pending``) of so many rows reads them in
        the packed layout (kernels.PackedRows): where the product takes the kernel for few rows."""
        key = (rows, dtype, pending)
        answer = self._accepts_packed.get(key)
        if answer is None:
            answer = kernels.takes_packed_rows(rows, self.weight, dtype)
            if pending and rows <= 64 and kernels.split_blocks(self.weight, dtype, rows) > 1:
                answer = True   # the partial products of few rows come from that kernel whatever the matrix
            self._accepts_packed[key] = answer
        return answer

    def forward_pending(self, x, residual):
        """residual + x W + b, as float32 rows or, where few rows meet few output columns and a long
        K, as rows whose sums are pending: the product cut along K into partial products, which
        whoever reads the rows next adds up (kernels.PendingRows)."""
        rows = x.shape[0]
        bucket = 0 if rows <= 64 else -(-rows // 128)  # the answer is the same inside a bucket
        k_blocks = self._split_blocks.get((bucket, x.dtype))
        if k_blocks is None:
            k_blocks = self._split_blocks[bucket, x.dtype] = kernels.split_blocks(self.weight, x.dtype, rows)
        if k_blocks > 1:
            return kernels.PendingRows(residual, kernels.linear_split(x, self.weight, k_blocks), self.bias)
        return self.forward(x, residual=residual)
