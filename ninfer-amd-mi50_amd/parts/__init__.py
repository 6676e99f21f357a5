from .attention import Attention
from .base import (Block, CacheNeed, CacheView, CallInfo, FeedForward, Mixer, Norm, Part,
                   PendingRows, PoolSpec, PositionEncoding, StepContext, WeightBinder, settle)
from .block import PreNormBlock
from .embedding import LMHead, TokenEmbedding
from .mlp import SwiGLU
from .moe import RoutedExperts, Routing, SoftmaxTopKRouter, SparseMoE, TopKRouter
from .norm import RMSNorm
from .rotary import NoPosition, Rotary

__all__ = ["Attention", "Block", "CacheNeed", "CacheView", "CallInfo", "FeedForward", "Mixer",
           "Norm", "Part", "PendingRows", "PoolSpec", "settle", "PositionEncoding", "StepContext", "WeightBinder", "PreNormBlock",
           "LMHead", "TokenEmbedding", "SwiGLU", "RoutedExperts", "Routing", "SoftmaxTopKRouter", "TopKRouter",
           "SparseMoE", "RMSNorm", "NoPosition", "Rotary"]
