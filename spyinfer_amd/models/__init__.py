from . import qwen3  # registers "Qwen3ForCausalLM"
from . import sefevik  # registers "Sefevik"
from .base import DecoderModel, LayerCall
