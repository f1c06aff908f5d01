from . import gimozen, gpt2  # register Gimozen and GPT2LMHeadModel
from .base import CacheGroupSpec, LayerCall, Model

__all__ = ["CacheGroupSpec", "LayerCall", "Model", "gimozen", "gpt2"]
