from . import qwen3  # registers the architecture
from .decoder import DecoderModel, LayerCall

__all__ = ["DecoderModel", "LayerCall"]
