"""Parts that models are put together from; see base.py for the interfaces."""

from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, CacheNeed, LayerCache,
                   Registry, StepContext)
from .linear import Linear
from .norm import LayerNorm, RMSNorm, ZeroCentredRMSNorm
from .rope import NoPositionEncoding, RotaryEncoding, RotaryFrequencies
from .attention import GQAAttention
from .mlp import GeluTanh, SquaredReLU, SwiGLU
from .lightning import LightningAttention
from .latent_attention import LatentAttention
from .streams import StreamConnection, StreamMixingBlock, StreamsResidual
from .block import PreNormBlock
from .embedding import CappedLMHead, Embedding, LMHead, ScaledEmbedding, ScaledLMHead
from .conv_attention import ConvGatedAttention
from .state_space import StateSpaceScan
from .experts import ClampedGLU, RoutedExperts
from .token_side import EmbeddingAgain, LoopInput, TokenSideInput, TokenSideTable
from .gated_attention import GatedAttention
from .mlstm import MatrixMemory
from .post_norm import PostNormBlock
from .gla import GatedLinearAttention
from .parallel import ParallelMixers

__all__ = ["BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITION_ENCODINGS", "CacheNeed", "LayerCache",
           "Registry", "StepContext", "Linear", "RMSNorm", "NoPositionEncoding", "RotaryEncoding",
           "GQAAttention", "SwiGLU", "PreNormBlock", "Embedding", "LMHead", "ZeroCentredRMSNorm", "RotaryFrequencies",
           "SquaredReLU", "LightningAttention", "LatentAttention", "StreamConnection", "StreamMixingBlock", "StreamsResidual",
           "ScaledLMHead", "LayerNorm", "CappedLMHead", "ScaledEmbedding", "ConvGatedAttention", "StateSpaceScan", "ClampedGLU",
           "RoutedExperts", "LoopInput", "TokenSideInput", "TokenSideTable", "GatedAttention", "MatrixMemory", "PostNormBlock",
           "GeluTanh", "GatedLinearAttention", "ParallelMixers", "EmbeddingAgain"]
