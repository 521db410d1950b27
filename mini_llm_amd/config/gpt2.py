"""Typed configuration of the GPT-2 architecture, read from its own config.json keys.

The reference fixes these numbers at compile time (engine/include/gpt2.h:12-19, the norm's
epsilon in engine/src/gpt2_gpu.cu:15); scripts/dump_reference.py:48-58 shows which config.json
keys they come from. Here they are data."""

from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError, ModelConfig, take_float, take_int

MAX_HEAD_SIZE = 256  # the widest head the attention kernels take (parts.attention.MAX_HEAD_SIZE)
ACTIVATIONS = ("gelu_new", "gelu")  # tanh form / exact erf form (engine/src/gelu.c:5-20)


@dataclass(frozen=True)
class GPT2Config(ModelConfig):
    n_layer: int
    n_embd: int
    n_head: int
    n_inner: int
    vocab_size: int
    n_positions: int
    layer_norm_epsilon: float
    activation_function: str
    eos_token_id: int | None = None

    @property
    def head_size(self) -> int:
        return self.n_embd // self.n_head

    @classmethod
    def from_dict(cls, raw: dict) -> "GPT2Config":
        n_embd = take_int(raw, "n_embd", 768)
        n_head = take_int(raw, "n_head", 12)
        if n_embd % n_head:
            raise ConfigError(f"n_embd={n_embd} is not divisible by n_head={n_head}")
        if n_embd // n_head > MAX_HEAD_SIZE:
            raise ConfigError(f"heads of {n_embd // n_head} (n_embd={n_embd} / n_head={n_head}) are wider than the attention kernels take: "
                              f"any size from 1 to {MAX_HEAD_SIZE} runs")
        # n_inner null or absent means four times the width (scripts/dump_reference.py:57)
        n_inner = raw.get("n_inner")
        n_inner = 4 * n_embd if n_inner is None else take_int(raw, "n_inner")
        activation = raw.get("activation_function", "gelu_new")
        if activation not in ACTIVATIONS:
            raise ConfigError(f"activation_function {activation!r} is not one of {ACTIVATIONS}")
        eps = take_float(raw, "layer_norm_epsilon", 1e-5)
        if not eps > 0:
            raise ConfigError(f"layer_norm_epsilon must be positive, not {eps}")
        # The formulas assume these; a file that says otherwise asks for another model.
        for key, needed in (
            ("tie_word_embeddings", True),
            ("scale_attn_weights", True),
            ("scale_attn_by_inverse_layer_idx", False),
            ("reorder_and_upcast_attn", False),
            ("add_cross_attention", False),
        ):
            if key in raw and bool(raw[key]) != needed:
                raise ConfigError(f"'{key}' = {raw[key]!r} is not supported (needs {needed})")
        eos = raw.get("eos_token_id")
        if eos is not None and (isinstance(eos, bool) or not isinstance(eos, int)):
            raise ConfigError(f"'eos_token_id' must be an integer or null, not {eos!r}")
        architectures = raw.get("architectures") or ["GPT2LMHeadModel"]
        return cls(
            architecture=architectures[0],
            n_layer=take_int(raw, "n_layer", 12),
            n_embd=n_embd,
            n_head=n_head,
            n_inner=n_inner,
            vocab_size=take_int(raw, "vocab_size", 50257),
            n_positions=take_int(raw, "n_positions", 1024),
            layer_norm_epsilon=eps,
            activation_function=activation,
            eos_token_id=eos,
        )

    def to_dict(self) -> dict:
        return {
            "architectures": [self.architecture],
            "model_type": "gpt2",
            "n_layer": self.n_layer,
            "n_embd": self.n_embd,
            "n_head": self.n_head,
            "n_inner": self.n_inner,
            "vocab_size": self.vocab_size,
            "n_positions": self.n_positions,
            "layer_norm_epsilon": self.layer_norm_epsilon,
            "activation_function": self.activation_function,
            "tie_word_embeddings": True,
            "eos_token_id": self.eos_token_id,
        }
