"""MI355X-native partition-overlap layer engine."""

from .block import DecoderLayer, LayerConfig, LayerStack

__all__ = ["DecoderLayer", "LayerConfig", "LayerStack"]
__version__ = "0.1.0"
