from .base import Part, Mixer, FeedForward, register_part, unregister_part, make_part, matrix_operand
from .norm import RMSNorm
from .position import RotaryEmbedding, NoPosition
from .attention import PagedAttention
from .ffn import GatedMLP
from .block import PreNormBlock
from .embedding import TokenEmbedding, LMHead
