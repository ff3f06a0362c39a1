from .base import (PAGE, Block, CacheSpec, FeedForward, Head, LayerCache, Mixer, Norm, ParamSpec, Part, Placement,
                   PositionEncoding, TokenEmbedding)
from .registry import LayerSpec, PartChoice, build_layer, make_part, register_part, registered
from .norm import RMSNorm
from .rope import RotaryEmbedding, inverse_frequencies
from .embedding import Embedding, OutputHead
from .mlp import GatedMLP
from .attention import Attention
from .block import PreNormBlock

__all__ = ["PAGE", "Block", "CacheSpec", "FeedForward", "LayerCache", "Mixer", "Norm", "ParamSpec", "Part",
           "Placement", "PositionEncoding", "TokenEmbedding", "Head", "LayerSpec", "PartChoice", "build_layer", "make_part",
           "register_part", "registered", "RMSNorm", "RotaryEmbedding", "inverse_frequencies", "Embedding",
           "OutputHead", "GatedMLP", "Attention", "PreNormBlock"]
