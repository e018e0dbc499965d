from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, CacheNeed, FeedForward,
                   HiddenStream, Mixer, Norm, Part, PartSpec, PositionEncoding, Registry, Runtime, TensorDecl,
                   Workspace, register_block, register_feed_forward, register_mixer, register_norm,
                   register_position_encoding)
from .plan import Call, EmbeddingSpec, HeadSpec, LayerPlan, ModelPlan, TensorLocation
from .norm import RMSNorm, RMSNormSpec
from .rope import RotaryEmbedding, RotarySpec, inverse_frequencies
from .attention import Attention, AttentionSpec
from .mlp import SwiGLU, SwiGLUSpec
from .block import PreNormBlock, PreNormBlockSpec
