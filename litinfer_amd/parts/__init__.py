from .base import (BatchNeeds, Block, FeedForward, Mixer, Norm, PagedKVNeed, PagedNeed, PagedTensor, Part,
                   Runtime, StateNeed, build_part, needs_of, register_part)
from .position import Position, RopeNeox, RopePairs
from .linear import Linear
from .stream import BranchStream, ResidualStream
from .norm import LayerNorm, RMSNorm
from .attention import GQAttention
from .masked_attention import LatentAttention, MaskedAttention
from .mlp import GeluMLP, ReluSquaredMLP, SwiGLUMLP
from .moe import RoutedMLP, RoutedReluSquaredMLP
from .mamba2 import Mamba2Mixer
from .diff_attention import DiffAttention
from .delta import GatedDeltaMixer
from .retention import RetentionMixer
from .mixer_pair import MixerPair
from .block import ParallelBlock, PreNormBlock, SandwichBlock
from .token_side import TokenSideInput
from .inject import LoopEntry, LoopMix
from .embedding import LinearHead, PairHashEmbedding, TokenEmbedding

__all__ = ["BatchNeeds", "Block", "FeedForward", "Mixer", "Norm", "PagedKVNeed", "PagedNeed", "PagedTensor",
           "Part", "Runtime", "StateNeed", "needs_of",
           "build_part", "register_part", "Position", "RopeNeox", "Linear", "ResidualStream", "RMSNorm",
           "GQAttention", "SwiGLUMLP", "PreNormBlock", "LinearHead", "TokenEmbedding", "RopePairs", "BranchStream",
           "MaskedAttention", "LatentAttention", "RoutedReluSquaredMLP", "Mamba2Mixer", "DiffAttention", "ReluSquaredMLP", "SandwichBlock", "TokenSideInput", "LoopEntry", "LoopMix", "LayerNorm", "GeluMLP", "RoutedMLP", "ParallelBlock", "PairHashEmbedding", "GatedDeltaMixer",
           "RetentionMixer", "MixerPair"]
