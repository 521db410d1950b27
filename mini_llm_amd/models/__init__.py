from . import gpt2  # registers GPT2LMHeadModel
from .base import CacheGroupSpec, LayerCall, Model

__all__ = ["CacheGroupSpec", "LayerCall", "Model", "gpt2"]
