from .base import Part, collect_params
from .norm import RMSNorm
from .position import RotaryPosition, NoPosition
from .attention import Attention
from .feed_forward import GatedMLP
from .embedding import Embedding, LMHead
from .block import Block, PreNormBlock, SubLayer

__all__ = ["Part", "collect_params", "RMSNorm", "RotaryPosition", "NoPosition", "Attention", "GatedMLP",
           "Embedding", "LMHead", "Block", "PreNormBlock", "SubLayer"]
