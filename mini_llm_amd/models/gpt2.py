"""The GPT-2 architecture as a recipe of parts, chosen by its configuration.

Tensor names are those of the reference's weight files (engine/src/gpt2.c:34-108,131-137), with
or without the ``transformer.`` prefix."""

from __future__ import annotations

import math

from ..config.gpt2 import GPT2Config
from ..config.registry import register_architecture
from ..parts import TiedHead, TokenEmbedding, make_part
from .base import LayerCall, Model


class GPT2Model(Model):
    def canonical_tensor_name(self, name: str):
        if name.startswith("transformer."):
            name = name[len("transformer."):]
        # causal-mask buffers of older files, and the head that is tied to wte
        if name.endswith(".attn.bias") or name.endswith(".attn.masked_bias") or name == "lm_head.weight":
            return None
        return name


def build_gpt2(config: GPT2Config, precision) -> GPT2Model:
    width = config.n_embd
    # the two projections into the residual stream are drawn narrower, by the depth
    residual_std = 0.02 / math.sqrt(2 * config.n_layer)
    blocks = []
    for _ in range(config.n_layer):
        blocks.append(make_part(
            "block", "pre_norm",
            norm_1=make_part("norm", "layernorm", width=width, eps=config.layer_norm_epsilon),
            mixer=make_part("mixer", "causal_attention", width=width, n_heads=config.n_head, out_std=residual_std),
            norm_2=make_part("norm", "layernorm", width=width, eps=config.layer_norm_epsilon),
            feed_forward=make_part("feed_forward", "dense_mlp", width=width, inner=config.n_inner,
                                   activation=config.activation_function, down_std=residual_std),
            compute_dtype=precision.compute,
        ))
    embedding = TokenEmbedding(config.vocab_size, width)
    return GPT2Model(
        config, precision,
        embedding=embedding,
        position_encoding=make_part("position_encoding", "learned", n_positions=config.n_positions, width=width),
        blocks=blocks,
        schedule=[LayerCall(block=i, cache=i) for i in range(config.n_layer)],
        final_norm=make_part("norm", "layernorm", width=width, eps=config.layer_norm_epsilon),
        head=TiedHead(embedding),
        names={"embedding": "wte.", "position_encoding": "wpe.", "block": "h.{i}.", "final_norm": "ln_f."},
    )


register_architecture("GPT2LMHeadModel", GPT2Config, build_gpt2)
