from .base import Part, Mixer, FeedForward, register_part, unregister_part, make_part, matrix_operand, CAST
from .norm import RMSNorm, LayerNorm
from .position import RotaryEmbedding, NoPosition
from .attention import PagedAttention, NormedGatedAttention, LatentAttention, SigmoidAttention
from .recurrent import GatedLinearAttention, StateSpaceDuality, SideBySide, GatedDeltaRule, MinGRU
from .ffn import GatedMLP, ClampedGLU, DenseMLP, RoutedExperts
from .block import PreNormBlock, SandwichBlock, PostNormBlock, NormedMean
from .embedding import TokenEmbedding, PairHashEmbedding, LMHead
