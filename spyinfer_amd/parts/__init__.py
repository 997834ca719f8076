from .attention import PagedAttention
from .base import Block, FeedForward, Mixer, Norm, Part, PositionEncoding
from .block import PreNormBlock
from .embedding import LMHead, TokenEmbedding
from .mlp import GatedMLP
from .norm import RMSNorm
from .rotary import RotaryEmbedding
