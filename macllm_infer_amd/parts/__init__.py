from .base import BuildContext, FeedForward, Mixer, Part, Residual, part_class, register_part
from .block import ParallelPreNormBlock, arrangement_class, register_arrangement, register_fusion
from .linear import Linear
from .norm import RmsNorm
from .position import NoPosition, PositionEncoding, Rope
from .attention import Attention
from .mamba2 import Mamba2
from .ffn import SwiGLU
from . import fused          # registers the fast paths of the layer arrangements
from .fused import FastPathDeclined

__all__ = ["Attention", "BuildContext", "FastPathDeclined", "FeedForward", "Linear", "Mamba2", "Mixer", "NoPosition", "Part",
           "ParallelPreNormBlock", "PositionEncoding", "Residual", "RmsNorm", "Rope", "SwiGLU",
           "arrangement_class", "part_class", "register_arrangement", "register_fusion", "register_part"]
