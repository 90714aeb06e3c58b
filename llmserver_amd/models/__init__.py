from . import barotar, gogalix, kerudra, qwen3, zepolix  # registers the architectures
from .decoder import DecoderModel, LayerCall

__all__ = ["DecoderModel", "LayerCall"]
