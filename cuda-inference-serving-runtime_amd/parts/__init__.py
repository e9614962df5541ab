from .base import Part, Mixer, FeedForward, register_part, unregister_part, make_part, matrix_operand, CAST
from .norm import RMSNorm, LayerNorm
from .position import RotaryEmbedding, NoPosition
from .attention import PagedAttention, NormedGatedAttention, LatentAttention, SigmoidAttention, TalkingAttention
from .recurrent import GatedLinearAttention, StateSpaceDuality, SideBySide, GatedDeltaRule, MinGRU, MatrixMemory
from .ffn import GatedMLP, ClampedGLU, DenseMLP, RoutedExperts, ScoredExperts
from .block import PreNormBlock, SandwichBlock, PostNormBlock, NormedMean, ScaledSum
from .embedding import TokenEmbedding, PairHashEmbedding, LMHead
