from .attention import Attention
from .base import (Block, CacheNeed, CacheView, CallInfo, FeedForward, Mixer, Norm, Part,
                   PendingRows, PoolSpec, PositionEncoding, StepContext, WeightBinder, settle)
from .block import OutputNormBlock, ParallelBlock, PreNormBlock, SandwichBlock
from .diff_attention import DifferentialAttention
from .embedding import LMHead, TokenEmbedding
from .gla import GatedLinearAttention
from .latent_attention import LatentAttention
from .lightning import LightningAttention
from .mlp import MLP, SwiGLU
from .moe import RoutedExperts, Routing, SoftmaxTopKRouter, SparseMoE, TopKRouter
from .norm import LayerNorm, OutputLayerNorm, OutputRMSNorm, RMSNorm
from .rotary import NoPosition, Rotary
from .reentry import StreamReentry
from .short_conv import ShortConv
from .sigmoid_attention import SigmoidAttention

__all__ = ["Attention", "Block", "CacheNeed", "CacheView", "CallInfo", "FeedForward", "Mixer",
           "Norm", "Part", "PendingRows", "PoolSpec", "settle", "PositionEncoding", "StepContext", "WeightBinder", "PreNormBlock",
           "LMHead", "TokenEmbedding", "SwiGLU", "RoutedExperts", "Routing", "SoftmaxTopKRouter", "TopKRouter",
           "SparseMoE", "RMSNorm", "NoPosition", "Rotary", "OutputNormBlock", "OutputRMSNorm",
           "LatentAttention", "LightningAttention", "ShortConv", "ParallelBlock",
           "DifferentialAttention", "MLP", "StreamReentry", "GatedLinearAttention",
           "SigmoidAttention", "SandwichBlock", "LayerNorm", "OutputLayerNorm"]
