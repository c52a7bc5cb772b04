from .model import DecoderModel, LayerCall
from . import llama  # registers "LlamaForCausalLM"
from . import rilonex  # registers "Rilonex"
from . import bidirax  # registers "Bidirax"
from . import zetonex  # registers "Zetonex"

__all__ = ["DecoderModel", "LayerCall", "llama", "rilonex", "bidirax", "zetonex"]
