from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, Block, CacheNeed,
                   Embedding, FeedForward, Head, HiddenStream, KeepAll, KeepWindow, KeyValueNeed, Mixer, Norm, Part,
                   PartSpec, PositionEncoding, Registry, Retention, Runtime, TensorDecl, Workspace, register_block,
                   register_embedding, register_feed_forward, register_head, register_mixer, register_norm,
                   register_position_encoding)
from .plan import Call, EmbeddingSpec, HeadSpec, LayerPlan, ModelPlan, TensorLocation
from .norm import RMSNorm, RMSNormSpec
from .rope import RotaryEmbedding, RotarySpec, inverse_frequencies
from .attention import Attention, AttentionSpec
from .mlp import SwiGLU, SwiGLUSpec
from .block import PreNormBlock, PreNormBlockSpec
from .io import LinearHead, TokenEmbedding
