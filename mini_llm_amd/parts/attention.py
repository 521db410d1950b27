"""Causal multi-head attention over the paged cache, with a fused q/k/v projection.

Formulas in the reference's order: q, k, v are column blocks of one product
(engine/src/gpt2.c:79-90); head h owns columns [h*hs, (h+1)*hs) (engine/src/attention.c:78-97);
scores scaled by 1/sqrt(head size), causal, softmax in 32-bit (engine/src/attention.cu:90-123);
the output projection adds its bias and the residual (engine/src/transformer_block.c:60-62)."""

from __future__ import annotations

import math

import torch

from ..ops import kernels
from .base import KVNeed, LayerContext, Mixer, register_part
from .linear import Linear
from .norms import LayerNorm


# The widest head any attention kernel takes (the general kernel keeps a head's output in four
# registers a lane). Heads of 16 to 128 in steps of 16 take the matrix-core kernel in prompt
# portions and powers of two the split-key kernel in decoding; every other size runs through the
# general kernel, a wave per (token, head).
MAX_HEAD_SIZE = 256


class CausalSelfAttention(Mixer):
    graph_safe = True
    short_portion = kernels.DECODE_MAX_Q_LEN   # what the split-key kernel takes
    decode_reaches = kernels.DECODE_LAYER_REACHES

    def __init__(self, width: int, n_heads: int, n_kv_heads: int | None = None, head_size: int | None = None,
                 window: int | None = None, out_std: float = 0.02, qkv_name: str = "c_attn.", out_name: str = "c_proj."):
        self.width, self.n_heads = width, n_heads
        self.n_kv_heads = n_heads if n_kv_heads is None else n_kv_heads
        self.head_size = width // n_heads if head_size is None else head_size
        if self.n_heads % self.n_kv_heads:
            raise ValueError(f"{n_heads} heads do not divide into {self.n_kv_heads} key/value heads")
        if not 1 <= self.head_size <= MAX_HEAD_SIZE:
            raise ValueError(f"head size {self.head_size} is not in 1..{MAX_HEAD_SIZE}")
        self.window = window
        self.scale = 1.0 / math.sqrt(self.head_size)
        self.q_width = self.n_heads * self.head_size
        self.kv_width = self.n_kv_heads * self.head_size
        self.qkv = Linear(width, self.q_width + 2 * self.kv_width)
        self.out = Linear(self.q_width, width, weight_std=out_std)
        self._names = (qkv_name, out_name)

    def children(self):
        return {self._names[0]: self.qkv, self._names[1]: self.out}

    def kv_need(self):
        return KVNeed(self.n_kv_heads, self.head_size, self.window)

    def _fused_qkv(self, ctx: LayerContext, dtype) -> bool:
        """One kernel projects, keeps q and puts keys and values into their pages."""
        page_size = ctx.k_pages.shape[2]
        return bool(ctx.write_cache and self.width % (16 // (4 if dtype == torch.float32 else 2)) == 0 and page_size & (page_size - 1) == 0)

    def forward(self, x, residual, ctx: LayerContext):
        """x: plain rows, or kernels.PackedRows where ``forward_normed`` asked the norm for them."""
        rows = x.shape[0]
        if self._fused_qkv(ctx, x.dtype):
            q = kernels.linear_qkv_cache(x, self.qkv.weight, self.qkv.bias, ctx.k_pages, ctx.v_pages, ctx.group.slots,
                                         self.n_heads, self.n_kv_heads, self.head_size)
        else:
            qkv = self.qkv.forward(x)
            q = qkv[:, : self.q_width]
            if ctx.write_cache:
                k = qkv[:, self.q_width : self.q_width + self.kv_width]
                v = qkv[:, self.q_width + self.kv_width :]
                kernels.cache_write(k, v, ctx.k_pages, ctx.v_pages, ctx.group.slots, self.n_kv_heads, self.head_size)
        mixed = kernels.paged_attention(
            q, ctx.k_pages, ctx.v_pages, ctx.batch.token_request, ctx.batch.positions, ctx.group.block_tables,
            self.n_heads, self.n_kv_heads, self.head_size, self.scale, window=self.window or 0,
            max_q_len=ctx.batch.max_q_len, max_len=ctx.batch.max_total_len,
            q_starts=ctx.batch.q_starts, context_lens=ctx.batch.context_lens, first_row=getattr(ctx.batch, "first_row", 0),
            # few rows: the output product reads them faster in the packed layout
            packed_out=kernels.PACKED_ROWS_FROM <= rows <= 64 and self.out.accepts_packed_rows(rows, q.dtype, pending=True),
            **({"short_rows": ctx.batch.short_rows, "short_requests": ctx.batch.short_requests}
               if ctx.batch.short_portion <= kernels.DECODE_MAX_Q_LEN else {}),
        )
        return self.out.forward_pending(mixed, residual)

    def forward_normed(self, hidden, norm, compute_dtype, ctx: LayerContext):
        # rows that are each the newest token of their request: the whole chain in one kernel, while a block of it can
        # walk a row's keys alone (past that the kernel that spreads a row's keys over many blocks is worth its company)
        if (ctx.batch.max_q_len == 1 and ctx.batch.max_total_len <= kernels.decode_layer_reach(hidden.shape[0]) and hidden.shape[0] <= kernels.layer_kernel_rows(self.width) and isinstance(norm, LayerNorm)
                and isinstance(self.qkv.weight, kernels.PackedMatrix) and isinstance(self.out.weight, kernels.PackedMatrix)
                and self.qkv.weight.dtype == torch.bfloat16 and ctx.k_pages.dtype == torch.bfloat16
                and kernels.decode_layer_supported(self.width, self.head_size, ctx.k_pages.shape[2])):
            return kernels.decode_attention_half(
                hidden, norm.weight, norm.bias, norm.eps, self.qkv.weight, self.qkv.bias, self.out.weight, self.out.bias,
                ctx.k_pages, ctx.v_pages, ctx.group.slots, ctx.batch.token_request, ctx.batch.positions, ctx.group.block_tables,
                self.n_heads, self.n_kv_heads, self.head_size, self.scale, window=self.window or 0, write_cache=ctx.write_cache)
        # kernel by kernel; few rows go from the norm to the q/k/v product in the packed layout
        rows = hidden.shape[0]
        packed = kernels.PACKED_ROWS_FROM <= rows <= 64 and self._fused_qkv(ctx, compute_dtype) and self.qkv.accepts_packed_rows(rows, compute_dtype)
        x, hidden = norm.forward_with_sums(hidden, compute_dtype, packed=packed)
        return self.forward(x, hidden, ctx)


register_part("mixer", "causal_attention", CausalSelfAttention)
