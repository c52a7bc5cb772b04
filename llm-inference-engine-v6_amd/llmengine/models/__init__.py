from .model import DecoderModel, LayerCall
from . import llama  # registers "LlamaForCausalLM"
from . import rilonex  # registers "Rilonex"
from . import bidirax  # registers "Bidirax"
from . import zetonex  # registers "Zetonex"
from . import zapolorn  # registers "Zapolorn"

__all__ = ["DecoderModel", "LayerCall", "llama", "rilonex", "bidirax", "zetonex", "zapolorn"]
