from .base import (
    BLOCKS,
    CONNECTIONS,
    EMBEDDINGS,
    FEED_FORWARDS,
    HEADS,
    MIXERS,
    NORMS,
    POSITION_ENCODINGS,
    Block,
    CacheSpec,
    ChunkedKVSpec,
    Connection,
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
    TOKEN_INPUTS,
    TokenInput,
    register_part,
)
from . import norm, rope, attention, feedforward, block, embedding, token_shift, state_space, latent_attention, experts, connection, short_conv, token_side  # noqa: F401  (fill the registries)
from .linear import LinearWeights
from .norm import GroupRMSNorm, LayerNorm, RMSNorm, StreamRMSNorm, StreamUpdate
from .rope import NoPositionEncoding, RotaryEncoding, llama3_scale_frequencies, rotary_inverse_frequencies
from .attention import HeadNormAttention, PagedAttention, SideBySide, SinkAttention, TalkingAttention
from .feedforward import ActivatedMLP, GatedMLP, SwiGLU
from .block import ConnectedPreNormBlock, ParallelPreNormBlock, PostNormBlock, PreNormBlock, SharedNormParallelBlock
from .connection import HyperConnection, ResidualSum
from .embedding import LinearHead, NormedTokenEmbedding, TokenEmbedding
from .token_shift import TokenShift
from .state_space import GatedLinearAttention, MatrixMemory, SelectiveStateSpace
from .short_conv import InputConvolution
from .token_side import GatedTokenSide
from .latent_attention import LatentAttention
from .experts import RoutedExperts
