from .base import Part, Mixer, FeedForward, register_part, unregister_part, make_part, matrix_operand
from .norm import RMSNorm
from .position import RotaryEmbedding, NoPosition
from .attention import PagedAttention, NormedGatedAttention
from .recurrent import GatedLinearAttention, StateSpaceDuality, SideBySide
from .ffn import GatedMLP, ClampedGLU
from .block import PreNormBlock, SandwichBlock, NormedMean
from .embedding import TokenEmbedding, LMHead
