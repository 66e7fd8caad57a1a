from tokenmill_amd.parts.attention import GQAttention
from tokenmill_amd.parts.attention_latent import LatentAttention
from tokenmill_amd.parts.attention_sigmoid import SigmoidAttention
from tokenmill_amd.parts.attention_softmax import SoftmaxAttention
from tokenmill_amd.parts.base import (FeedForward, GroupStep, KVCacheSpec, KVCacheView, LayerCacheSpec, Mixer, Norm, NormedInput, Part,
                                      PositionEncoding, StateSpec, StateView, StepContext, as_tensor)
from tokenmill_amd.parts.block import GatedResidualBlock, PreNormBlock, SandwichBlock
from tokenmill_amd.parts.conv import ShortConvolution
from tokenmill_amd.parts.delta_rule import GatedDeltaRule
from tokenmill_amd.parts.embedding import LearnedPositions, OutputHead, TokenEmbedding
from tokenmill_amd.parts.gla import GatedLinearAttention
from tokenmill_amd.parts.linear import Linear
from tokenmill_amd.parts.mlp import DenseFeedForward, GatedFeedForward, SwiGLU
from tokenmill_amd.parts.moe import RoutedExperts, TableRoutedExperts
from tokenmill_amd.parts.parallel import ParallelMixer
from tokenmill_amd.parts.norm import GatedAdd, GroupRMSNorm, LayerNorm, PassThrough, RMSNorm
from tokenmill_amd.parts.position import NoPositionEncoding, RotaryEmbedding

__all__ = ["GQAttention", "FeedForward", "GroupStep", "KVCacheSpec", "KVCacheView", "Mixer", "Norm", "NormedInput", "as_tensor", "Part",
           "PositionEncoding", "StateSpec", "StateView", "StepContext", "PreNormBlock", "OutputHead",
           "TokenEmbedding", "Linear", "SwiGLU", "RMSNorm", "SigmoidAttention", "SandwichBlock", "LearnedPositions", "GatedLinearAttention",
           "DenseFeedForward", "GroupRMSNorm", "LatentAttention", "LayerCacheSpec", "GatedResidualBlock", "ShortConvolution",
           "TableRoutedExperts", "GatedAdd", "SoftmaxAttention", "RoutedExperts", "PassThrough", "LayerNorm", "NoPositionEncoding", "RotaryEmbedding",
           "GatedDeltaRule", "ParallelMixer", "GatedFeedForward"]
