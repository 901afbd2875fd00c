"""MI355X-native partition-overlap layer engine."""

from .block import DecoderLayer, LayerConfig, LayerStack
from .model import GPTModelShard, LanguageModelEmbedding

__all__ = ["DecoderLayer", "GPTModelShard", "LanguageModelEmbedding", "LayerConfig", "LayerStack"]
__version__ = "0.1.0"
