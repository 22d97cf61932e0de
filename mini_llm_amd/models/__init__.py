from . import gimozen, gpt2, ketolix, perezen  # register Gimozen, GPT2LMHeadModel, Ketolix and Perezen
from .base import CacheGroupSpec, LayerCall, Model

__all__ = ["CacheGroupSpec", "LayerCall", "Model", "gimozen", "gpt2", "ketolix", "perezen"]
