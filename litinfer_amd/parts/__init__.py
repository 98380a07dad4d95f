from .base import (BatchNeeds, Block, FeedForward, Mixer, Norm, PagedKVNeed, PagedNeed, PagedTensor, Part,
                   Runtime, StateNeed, build_part, needs_of, register_part)
from .position import Position, RopeNeox, RopePairs
from .linear import Linear
from .stream import BranchStream, ResidualStream
from .norm import RMSNorm
from .attention import GQAttention
from .masked_attention import LatentAttention, MaskedAttention
from .mlp import ReluSquaredMLP, SwiGLUMLP
from .moe import RoutedReluSquaredMLP
from .mamba2 import Mamba2Mixer
from .diff_attention import DiffAttention
from .block import PreNormBlock, SandwichBlock
from .token_side import TokenSideInput
from .inject import LoopEntry
from .embedding import LinearHead, TokenEmbedding

__all__ = ["BatchNeeds", "Block", "FeedForward", "Mixer", "Norm", "PagedKVNeed", "PagedNeed", "PagedTensor",
           "Part", "Runtime", "StateNeed", "needs_of",
           "build_part", "register_part", "Position", "RopeNeox", "Linear", "ResidualStream", "RMSNorm",
           "GQAttention", "SwiGLUMLP", "PreNormBlock", "LinearHead", "TokenEmbedding", "RopePairs", "BranchStream",
           "MaskedAttention", "LatentAttention", "RoutedReluSquaredMLP", "Mamba2Mixer", "DiffAttention", "ReluSquaredMLP", "SandwichBlock", "TokenSideInput", "LoopEntry"]
