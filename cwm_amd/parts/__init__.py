from .base import (
    BLOCKS,
    EMBEDDINGS,
    FEED_FORWARDS,
    HEADS,
    MIXERS,
    NORMS,
    POSITION_ENCODINGS,
    Block,
    CacheSpec,
    Embedding,
    FeedForward,
    Head,
    LayerCall,
    LayerPlan,
    Mixer,
    ModelPlan,
    Norm,
    PagedKVSpec,
    Part,
    PartChoice,
    PartSlot,
    PositionEncoding,
    Runtime,
    StateSpec,
    TensorSpec,
    register_part,
)
from . import norm, rope, attention, feedforward, block, embedding  # noqa: F401  (fill the registries)
from .linear import LinearWeights
from .norm import RMSNorm
from .rope import NoPositionEncoding, RotaryEncoding, llama3_scale_frequencies, rotary_inverse_frequencies
from .attention import PagedAttention
from .feedforward import SwiGLU
from .block import PreNormBlock
from .embedding import LinearHead, TokenEmbedding
