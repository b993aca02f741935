from .decoder import DecoderModel, LayerRun, TokenEmbedding, OutputHead
from .qwen3 import build_qwen3

__all__ = ["DecoderModel", "LayerRun", "TokenEmbedding", "OutputHead", "build_qwen3"]
