from .attention import GroupedQueryAttention
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, FeedForward,
                   Hidden, Mixer, Norm, Part, PositionEncoding, make_part, register_part)
from .block import ConvInputBlock, HyperConnectionBlock, OutputNormBlock, PreNormBlock
from .diff_attention import DifferentialAttention
from .embedding import OutputHead, TokenEmbedding
from .feed_forward import SwiGLU
from .gated_unit import RealGatedUnit
from .group_norm import GroupRMSNorm
from .input_conv import ShortInputConv
from .latent_attention import LatentAttention
from .linear import Linear
from .linear_attention import (BonusTimeMixing, FixedDecayAttention, GatedDeltaRule,
                               GatedLinearAttention)
from .mingru import MinGRU
from .moe import MixtureOfExperts
from .norm import LayerNorm, RMSNorm
from .parallel import ParallelMixer
from .passes import PassEntry
from .positions import LearnedPositions
from .rotary import RotaryEncoding, Rotation
from .scored_attention import ScoredAttention
from .shortconv import GatedShortConv

__all__ = ["GroupedQueryAttention", "BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS",
           "POSITION_ENCODINGS", "Block", "FeedForward", "Hidden", "Mixer", "Norm", "Part",
           "PositionEncoding", "make_part", "register_part", "PreNormBlock", "OutputHead",
           "TokenEmbedding", "SwiGLU", "Linear", "RMSNorm", "RotaryEncoding", "Rotation",
           "GatedShortConv", "ConvInputBlock", "DifferentialAttention", "GroupRMSNorm",
           "ShortInputConv", "MinGRU", "MixtureOfExperts", "LearnedPositions", "OutputNormBlock",
           "LatentAttention", "GatedDeltaRule", "GatedLinearAttention", "ParallelMixer",
           "ScoredAttention", "RealGatedUnit", "BonusTimeMixing", "FixedDecayAttention",
           "PassEntry", "HyperConnectionBlock", "LayerNorm"]
