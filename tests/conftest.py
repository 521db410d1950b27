"""Shared fixtures: the two tiny GPT-2 configurations and model folders made in temp folders."""

import json
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))
if str(ROOT / "tests") not in sys.path:
    sys.path.insert(0, str(ROOT / "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


# Two tiny configurations that differ in every size and option.
TINY_A = {
    "architectures": ["GPT2LMHeadModel"],
    "model_type": "gpt2",
    "n_layer": 2,
    "n_embd": 64,
    "n_head": 4,
    "n_inner": None,
    "vocab_size": 512,
    "n_positions": 128,
    "layer_norm_epsilon": 1e-5,
    "activation_function": "gelu_new",
    "tie_word_embeddings": True,
}
TINY_B = {
    "architectures": ["GPT2LMHeadModel"],
    "model_type": "gpt2",
    "n_layer": 3,
    "n_embd": 96,
    "n_head": 3,
    "n_inner": 320,
    "vocab_size": 1000,
    "n_positions": 64,
    "layer_norm_epsilon": 1e-6,
    "activation_function": "gelu",
    "tie_word_embeddings": True,
}
# A third one for long sequences: head size 48 (no power of two), several pages of context.
TINY_C = {
    "architectures": ["GPT2LMHeadModel"],
    "model_type": "gpt2",
    "n_layer": 2,
    "n_embd": 240,
    "n_head": 5,
    "n_inner": 200,
    "vocab_size": 777,
    "n_positions": 600,
    "layer_norm_epsilon": 3e-5,
    "activation_function": "gelu_new",
    "tie_word_embeddings": True,
}
# Sizes no kernel's fast path takes: heads of 14 (no multiple of 16), a width and hidden units that
# are no multiple of four, an odd vocabulary.
TINY_D = {
    "architectures": ["GPT2LMHeadModel"],
    "model_type": "gpt2",
    "n_layer": 2,
    "n_embd": 42,
    "n_head": 3,
    "n_inner": 75,
    "vocab_size": 301,
    "n_positions": 96,
    "layer_norm_epsilon": 2e-5,
    "activation_function": "gelu",
    "tie_word_embeddings": True,
}
# Heads of 24 and hidden units that are a multiple of four but not of eight: the down product's K is
# a whole number of 16-byte pieces in 32-bit and not in bfloat16.
TINY_E = {
    "architectures": ["GPT2LMHeadModel"],
    "model_type": "gpt2",
    "n_layer": 3,
    "n_embd": 72,
    "n_head": 3,
    "n_inner": 100,
    "vocab_size": 409,
    "n_positions": 160,
    "layer_norm_epsilon": 1e-5,
    "activation_function": "gelu_new",
    "tie_word_embeddings": True,
}
TINY = {"A": (TINY_A, 0), "B": (TINY_B, 2), "C": (TINY_C, 8), "D": (TINY_D, 11), "E": (TINY_E, 12)}


def sharpen_attention(weights: dict, config: dict, factor: float = 8.0) -> None:
    """With the benchmark's init the scores are a few hundredths and every softmax is nearly
    uniform: keys could be swapped or a page mixed up and the logits would hardly move. The query
    and key columns of c_attn are scaled up so that attention weights differ by orders of
    magnitude and a wrong key shows."""
    d = config["n_embd"]
    for i in range(config["n_layer"]):
        weights[f"h.{i}.attn.c_attn.weight"][:, : 2 * d] *= factor
        weights[f"h.{i}.attn.c_attn.bias"][: 2 * d] *= factor


def make_plain_model_dir(path: Path, config: dict, seed: int, bf16: bool = False, prefix: str = "transformer."):
    """A model folder written by the plain implementation's own writer."""
    import plain_gpt2

    path.mkdir(parents=True, exist_ok=True)
    weights = plain_gpt2.random_weights(config, seed)
    sharpen_attention(weights, config)
    (path / "config.json").write_text(json.dumps(config))
    plain_gpt2.write_safetensors(
        path / "model.safetensors", {prefix + k: v for k, v in weights.items()}, bf16=bf16
    )
    return weights


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """name -> (folder, config, float32 weights) for the tiny configurations (float32 files)."""
    out = {}
    for name, (config, seed) in TINY.items():
        folder = tmp_path_factory.mktemp(f"tiny_{name}")
        weights = make_plain_model_dir(folder, config, seed)
        out[name] = (folder, dict(config), weights)
    return out


def random_tokens(seed: int, n: int, vocab: int):
    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()
