from .base import (PAGE, Block, CacheSpec, FeedForward, Head, LayerCache, Mixer, Norm, ParamSpec, Part, Placement,
                   PositionEncoding, TokenEmbedding)
from .registry import LayerSpec, PartChoice, build_layer, make_part, register_part, registered
from .norm import CenteredRMSNorm, RMSNorm
from .rope import RotaryEmbedding, inverse_frequencies
from .embedding import Embedding, OutputHead
from .mlp import GatedMLP
from .attention import Attention
from .block import OutputNormBlock, ParallelBlock, PreNormBlock, SandwichBlock
from .projected import ParallelMixer, ProjectedMixer
from .rglru import RGLRU
from .delta import GatedDeltaRule
from .sigmoid_attention import SigmoidAttention
from .hyper import HyperConnectionBlock
from .latent_attention import LatentAttention
from .moe import MixtureOfExperts
from .window_attention import WindowAttention
from .linear_attention import GatedLinearAttention
from .reentry import PassInput

__all__ = ["PAGE", "Block", "CacheSpec", "FeedForward", "LayerCache", "Mixer", "Norm", "ParamSpec", "Part",
           "Placement", "PositionEncoding", "TokenEmbedding", "Head", "LayerSpec", "PartChoice", "build_layer", "make_part",
           "register_part", "registered", "RMSNorm", "RotaryEmbedding", "inverse_frequencies", "Embedding",
           "OutputHead", "GatedMLP", "Attention", "PreNormBlock", "ParallelMixer", "ProjectedMixer", "RGLRU", "GatedDeltaRule",
           "SigmoidAttention", "HyperConnectionBlock", "CenteredRMSNorm", "SandwichBlock", "LatentAttention",
           "MixtureOfExperts", "WindowAttention", "PassInput", "ParallelBlock", "OutputNormBlock", "GatedLinearAttention"]
