from .model import DecoderModel, LayerCall
from . import llama  # registers "LlamaForCausalLM"

__all__ = ["DecoderModel", "LayerCall", "llama"]
