from .registry import register_part, unregister_part, part_class, build_part, FAMILIES
from .base import (Part, Norm, NormedInput, PendingSums, PositionEncoding, Mixer, FeedForward, Block,
                   KVCacheSpec, CacheSpec, PageTensor)
from .norms import RMSNorm
from .positions import RotaryEmbedding, NoPosition
from .attention import GQAAttention
from .feed_forward import SwiGLU, interleave_gate_up
from .blocks import PreNormBlock, TokenEmbedding, LinearHead
