from . import dizizen, gimozen, gpt2, ketolix, perezen  # register Dizizen, Gimozen, GPT2LMHeadModel, Ketolix and Perezen
from .base import CacheGroupSpec, LayerCall, Model

__all__ = ["CacheGroupSpec", "LayerCall", "Model", "dizizen", "gimozen", "gpt2", "ketolix", "perezen"]
