from .model import DecoderModel, LayerCall
from . import llama  # registers "LlamaForCausalLM"
from . import rilonex  # registers "Rilonex"
from . import bidirax  # registers "Bidirax"

__all__ = ["DecoderModel", "LayerCall", "llama", "rilonex", "bidirax"]
