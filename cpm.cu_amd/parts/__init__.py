"""Parts a layer is put together from.  Importing this package registers the built-in kinds."""
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, FeedForward, Mixer, Norm, Part,
                   PartSpec, PositionEncoding, Registry, ResidualStream, Runtime, StepContext, WeightSpec, Workspace)
from .linear import Linear
from .norm import RMSNorm
from .rope import LongRotaryEncoding, RotaryEncoding
from .attention import GQAAttention, InfLLMv2Attention
from .ffn import GatedFFN
from .block import PreNormBlock
from .embedding import LMHead, TokenEmbedding
