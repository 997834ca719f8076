from . import qwen3  # registers "Qwen3ForCausalLM"
from .base import DecoderModel, LayerCall
