from .model import DecoderModel, LayerCall
from . import llama  # registers "LlamaForCausalLM"
from . import rilonex  # registers "Rilonex"

__all__ = ["DecoderModel", "LayerCall", "llama", "rilonex"]
