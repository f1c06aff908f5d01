from . import gimozen, gpt2, ketolix  # register Gimozen, GPT2LMHeadModel and Ketolix
from .base import CacheGroupSpec, LayerCall, Model

__all__ = ["CacheGroupSpec", "LayerCall", "Model", "gimozen", "gpt2", "ketolix"]
