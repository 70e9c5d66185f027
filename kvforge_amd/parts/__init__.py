from kvforge_amd.parts.base import (BLOCK, Block, CacheSpec, Embedding, FeedForward, Head, LayerCall,
                                    LayerState, Mixer, ModelSpec, Norm, PageTensor, Part, Positions, StateSpec,
                                    WeightSpec, attention_pages)
from kvforge_amd.parts.norm import NamedRMSNorm, OnePlusRMSNorm, RMSNorm, ScalarRMSNorm
from kvforge_amd.parts.positions import LearnedPositions, RotaryPositions, YarnStretch, scaled_inv_freq
from kvforge_amd.parts.attention import PagedAttention
from kvforge_amd.parts.feedforward import GatedFeedForward, PlainFeedForward, SwiGLU
from kvforge_amd.parts.side import TokenSideInput
from kvforge_amd.parts.mlstm import MatrixLSTM
from kvforge_amd.parts.moe import RoutedExperts
from kvforge_amd.parts.latent import LatentAttention
from kvforge_amd.parts.wkv import DecayMemory
from kvforge_amd.parts.linmem import LinearMemory
from kvforge_amd.parts.pair import MixerPair
from kvforge_amd.parts.embedding import LMHead, TokenEmbedding
from kvforge_amd.parts.block import ParallelBlock, PreNormBlock, SandwichBlock

__all__ = ["BLOCK", "PageTensor", "attention_pages", "Block", "CacheSpec", "Embedding", "FeedForward", "Head", "LayerCall", "LayerState", "Mixer", "ModelSpec",
           "Norm", "Part", "Positions", "StateSpec", "WeightSpec", "RMSNorm", "RotaryPositions",
           "scaled_inv_freq", "PagedAttention", "SwiGLU", "LMHead", "TokenEmbedding",
           "PreNormBlock", "ParallelBlock", "ScalarRMSNorm", "LearnedPositions", "GatedFeedForward",
           "TokenSideInput", "OnePlusRMSNorm", "YarnStretch", "MatrixLSTM", "RoutedExperts",
           "NamedRMSNorm", "LatentAttention", "DecayMemory", "SandwichBlock", "LinearMemory", "MixerPair",
           "PlainFeedForward"]
