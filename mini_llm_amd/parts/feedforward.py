"""Dense feed-forward: up projection, activation, down projection, residual sum
(engine/src/transformer_block.c:64-71). The activation is fused into the up product and the
residual sum into the down product."""

from __future__ import annotations

import torch

from ..ops import kernels
from .base import FeedForward, register_part
from .linear import Linear
from .norms import LayerNorm

ACTIVATIONS = ("gelu_new", "gelu")


class DenseMLP(FeedForward):
    def __init__(self, width: int, inner: int, activation: str, down_std: float = 0.02,
                 up_name: str = "c_fc.", down_name: str = "c_proj."):
        if activation not in ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not one of {ACTIVATIONS}")
        self.width, self.inner, self.activation = width, inner, activation
        self.up = Linear(width, inner)
        self.down = Linear(inner, width, weight_std=down_std)
        self._names = (up_name, down_name)

    def children(self):
        return {self._names[0]: self.up, self._names[1]: self.down}

    def forward(self, x, residual):
        return self.down.forward(self.up.forward(x, activation=self.activation), residual=residual)

    def forward_normed(self, hidden, norm, compute_dtype, ctx):
        # few rows: the whole chain in one kernel, cut along the hidden units
        if (hidden.shape[0] <= kernels.layer_kernel_rows(self.width) and ctx.batch.max_q_len == 1 and isinstance(norm, LayerNorm)
                and ctx.batch.max_total_len <= kernels.decode_layer_reach(hidden.shape[0])   # changes with the attention half
                and isinstance(self.up.weight, kernels.PackedMatrix) and isinstance(self.down.weight, kernels.PackedMatrix)
                and self.up.weight.dtype == torch.bfloat16 and kernels.decode_layer_supported(self.width, inner=self.inner)):
            return kernels.decode_mlp_half(hidden, norm.weight, norm.bias, norm.eps, self.up.weight, self.up.bias,
                                           self.down.weight, self.down.bias, activation=self.activation)
        # else kernel by kernel; the down product of few rows may come back with its sums pending, and
        # few rows go from kernel to kernel in the packed layout, which the products read faster
        rows = hidden.shape[0]
        few = kernels.PACKED_ROWS_FROM <= rows <= 64
        x, hidden = norm.forward_with_sums(hidden, compute_dtype, packed=few and self.up.accepts_packed_rows(rows, compute_dtype))
        packed_out = few and self.up.accepts_packed_rows(rows, compute_dtype) and self.down.accepts_packed_rows(rows, compute_dtype, pending=True)
        return self.down.forward_pending(self.up.forward(x, activation=self.activation, packed_out=packed_out), hidden)


register_part("feed_forward", "dense_mlp", DenseMLP)
