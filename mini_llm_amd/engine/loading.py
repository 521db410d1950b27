"""From a model folder to a model with weights on the GPU, and the cache that fits it."""

from __future__ import annotations

from ..cache import CacheManager
from ..config import get_architecture, load_config
from ..precision import Precision
from ..weights import bind_tensors, load_weights, random_tensors

DEFAULT_PAGE_SIZE = 64


def require_gpu(device="cuda:0"):
    import torch

    if not torch.cuda.is_available():
        raise RuntimeError("no GPU is visible: this engine has no CPU path")
    return torch.device(device)


def build_model(config, dtype):
    precision = Precision.from_name(dtype)
    return get_architecture(config.architecture).build(config, precision)


def load_model(model_dir, dtype, device="cuda:0"):
    """config.json chooses the architecture; model.safetensors fills its parts."""
    device = require_gpu(device)
    model = build_model(load_config(model_dir), dtype)
    load_weights(model, model_dir, device)
    return model


def random_model(config, seed: int, dtype, device="cuda:0"):
    """A model with random weights drawn as ``write_model_dir`` draws them, without a folder."""
    device = require_gpu(device)
    model = build_model(config, dtype)
    bind_tensors(model, random_tensors(model, seed), device)
    return model


def cache_bytes_per_token(groups, element_size: int) -> int:
    """What one token of one request takes in the page pools: a key row and a value row in every
    cache layer. (Every group's pool holds pages for the same number of tokens; a group with a
    window gives most of them back, but is sized like the others.)"""
    return sum(len(g.layers) * 2 * g.n_kv_heads * g.head_size * element_size for g in groups)


def tokens_for_memory(groups, element_size: int, gib: float, page_size: int) -> int:
    """The cache capacity in tokens (whole pages) that ``gib`` GiB of page pools hold."""
    per_token = cache_bytes_per_token(groups, element_size)
    if per_token == 0:
        raise ValueError("this model keeps no keys and values: its cache cannot be sized by memory")
    tokens = int(gib * (1 << 30)) // per_token // page_size * page_size
    if tokens < page_size:
        raise ValueError(f"{gib} GiB hold not even one page of {page_size} tokens ({per_token} bytes a token)")
    return tokens


def make_cache(model, *, max_tokens: int, page_size: int = DEFAULT_PAGE_SIZE, max_requests: int = 256, device="cuda:0",
               max_length: int | None = None):
    """A cache whose every group holds ``max_tokens`` tokens' worth of pages. ``max_length``: the
    longest sequence of one request (it sets the width of the block tables); by default the
    model's own position limit."""
    num_pages = max(1, -(-max_tokens // page_size))
    return CacheManager(
        model.cache_groups(), model.state_needs(), num_pages=num_pages, page_size=page_size, max_requests=max_requests,
        dtype=model.precision.compute, device=device, max_length=max_length if max_length is not None else model.max_positions(),
    )
