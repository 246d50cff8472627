from .base import Part, Mixer, FeedForward, register_part, unregister_part, make_part, matrix_operand
from .norm import RMSNorm, LayerNorm
from .position import RotaryEmbedding, NoPosition
from .attention import PagedAttention, NormedGatedAttention, LatentAttention
from .recurrent import GatedLinearAttention, StateSpaceDuality, SideBySide, GatedDeltaRule
from .ffn import GatedMLP, ClampedGLU, DenseMLP
from .block import PreNormBlock, SandwichBlock, NormedMean
from .embedding import TokenEmbedding, LMHead
