from .registry import register_part, unregister_part, part_class, build_part, FAMILIES
from .base import (Part, Norm, NormedInput, PendingSums, PositionEncoding, Mixer, FeedForward, Block,
                   KVCacheSpec, CacheSpec, PageTensor)
from .norms import RMSNorm, LayerNorm
from .positions import RotaryEmbedding, PairRotary, NoPosition
from .attention import GQAAttention, WindowedSinkAttention
from .linear_attention import GatedLinearAttention, DeltaRuleAttention
from .parallel import ParallelMixers
from .latent_attention import LatentAttention
from .feed_forward import SwiGLU, DenseFeedForward, interleave_gate_up
from .experts import RoutedExperts
from .blocks import PreNormBlock, SublayerNormBlock, SandwichNormBlock, GatedConvBlock, TokenEmbedding, PairHashEmbedding, LinearHead
