"""Arrangements of norm, mixer and feed-forward in a layer. GPT-2's is pre-norm: a norm before
the mixer and one before the feed-forward, each branch added to the residual stream
(engine/src/transformer_block.c:49-71)."""

from __future__ import annotations

from .base import Block, FeedForward, LayerContext, Mixer, Norm, register_part


class PreNormBlock(Block):
    def __init__(self, norm_1: Norm, mixer: Mixer, norm_2: Norm, feed_forward: FeedForward, compute_dtype,
                 names=("ln_1.", "attn.", "ln_2.", "mlp.")):
        self.norm_1, self.mixer, self.norm_2, self.feed_forward = norm_1, mixer, norm_2, feed_forward
        self.compute_dtype = compute_dtype
        self._names = names

    def children(self):
        return dict(zip(self._names, (self.norm_1, self.mixer, self.norm_2, self.feed_forward)))

    def mixer_part(self):
        return self.mixer

    takes_pending = True

    def forward(self, hidden, ctx: LayerContext):
        hidden = self.mixer.forward_normed(hidden, self.norm_1, self.compute_dtype, ctx)
        return self.feed_forward.forward_normed(hidden, self.norm_2, self.compute_dtype, ctx)


register_part("block", "pre_norm", PreNormBlock)
