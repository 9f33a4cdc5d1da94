"""Parts that layers are put together from: mixers, feed-forwards, norms, position encodings,
and the arrangement of a block."""

from .base import (Block, Convolution, FeedForward, HiddenState, Mixer, Norm, ParamDecl, Part, PositionEncoding,
                   known_parts, make_part, prepare_parts, register_part)
from .attention import AttentionPlanner, GQAttention
from .block import BranchNormBlock, ParallelBlock, PreNormBlock, SandwichNormBlock
from .conv import CausalResidualConvolution
from .embedding import LMHead, PairHashEmbedding, TokenEmbedding
from .latent_attention import LatentAttention
from .linear import Linear
from .linear_attention import GatedLinearAttention
from .mlp import SwiGLU
from .mlstm import MLSTM
from .moe import RoutedExperts
from .norm import GroupRMSNorm, LayerNorm, RMSNorm, StreamReader
from .retention import Retention, SideBySide
from .rope import NoPositionEncoding, RotaryEncoding

__all__ = ["AttentionPlanner", "Block", "BranchNormBlock", "Retention", "SideBySide", "StreamReader", "CausalResidualConvolution", "Convolution", "GroupRMSNorm", "MLSTM", "RoutedExperts", "FeedForward", "GQAttention", "GatedLinearAttention", "HiddenState", "LMHead",
           "LatentAttention", "LayerNorm", "Linear", "PairHashEmbedding", "ParallelBlock", "SandwichNormBlock", "Mixer", "NoPositionEncoding", "Norm", "ParamDecl", "Part", "PositionEncoding",
           "PreNormBlock", "RMSNorm", "RotaryEncoding", "SwiGLU", "TokenEmbedding", "known_parts",
           "make_part", "prepare_parts", "register_part"]
