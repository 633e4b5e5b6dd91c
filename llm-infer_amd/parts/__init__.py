from .base import Part, collect_params
from .norm import LayerNorm, RMSNorm
from .position import HalfRotaryPosition, RotaryPosition, NoPosition
from .attention import Attention
from .feed_forward import DenseMLP, GatedMLP, PolyNormMLP, RoutedExperts
from .token_shift import ShiftedMixer
from .parallel import ParallelMixers
from .sigmoid_attention import SigmoidAttention
from .decay_attention import DecayLinearAttention
from .diff_attention import DifferentialAttention
from .state_space import SelectiveStateSpace
from .stream import DepthAverage, Reinject
from .embedding import BigramEmbedding, Embedding, LMHead
from .block import Block, ParallelBlock, PostNormBlock, PreNormBlock, SandwichBlock, SubLayer
from .short_conv import ConvMixer
from .latent_attention import LatentAttention
from .mlstm import MatrixLSTM
from .gated_attention import GatedAttention

__all__ = ["Part", "collect_params", "RMSNorm", "RotaryPosition", "NoPosition", "Attention", "GatedMLP",
           "Embedding", "LMHead", "Block", "PreNormBlock", "SubLayer", "LayerNorm", "PolyNormMLP", "ShiftedMixer",
           "ParallelMixers", "SigmoidAttention", "DecayLinearAttention", "PostNormBlock", "DifferentialAttention",
           "SelectiveStateSpace", "Reinject", "DenseMLP", "RoutedExperts", "DepthAverage", "BigramEmbedding", "ParallelBlock",
           "ConvMixer", "LatentAttention", "MatrixLSTM", "GatedAttention", "SandwichBlock", "HalfRotaryPosition"]
