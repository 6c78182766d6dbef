from .base import BuildContext, FeedForward, Mixer, Part, Residual, part_class, register_part
from .block import ParallelPreNormBlock, SandwichBlock, arrangement_class, register_arrangement, register_fusion
from .linear import Linear
from .norm import LayerNorm, RmsNorm
from .position import InterleavedRope, LogDistanceBias, NoPosition, PositionEncoding, Rope
from .attention import Attention
from .latent_attention import LatentAttention
from .mamba2 import Mamba2
from .ffn import PolyNormFFN, SwiGLU
from .moe import RoutedExperts
from .linear_state import GatedLinearAttention, GeneralDelta, Retention
from . import fused          # registers the fast paths of the layer arrangements
from .fused import FastPathDeclined

__all__ = ["Attention", "GatedLinearAttention", "BuildContext", "FastPathDeclined", "FeedForward", "GeneralDelta", "Linear", "LogDistanceBias", "Mamba2",
           "Mixer", "NoPosition", "Part", "PolyNormFFN", "Retention",
           "ParallelPreNormBlock", "SandwichBlock", "PositionEncoding", "Residual", "RmsNorm", "Rope", "SwiGLU",
           "arrangement_class", "part_class", "register_arrangement", "register_fusion", "register_part"]
