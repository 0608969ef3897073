from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITION_ENCODINGS, Block, CacheNeed,
                   Embedding, FeedForward, Head, HiddenStream, KeepAll, KeepChunks, KeepWindow, KeyValueNeed, Mixer, Norm, Part,
                   PartSpec, PositionEncoding, Registry, Retention, Runtime, TensorDecl, Workspace, register_block,
                   register_embedding, register_feed_forward, register_head, register_mixer, register_norm,
                   register_position_encoding)
from .plan import Call, EmbeddingSpec, HeadSpec, LayerPlan, ModelPlan, TensorLocation
from .norm import RMSNorm, RMSNormSpec
from .rope import RotaryEmbedding, RotarySpec, inverse_frequencies
from .attention import Attention, AttentionSpec
from .mlp import SwiGLU, SwiGLUSpec
from .block import PreNormBlock, PreNormBlockSpec, SandwichBlock, SandwichBlockSpec
from .delta_rule import DeltaRule, DeltaRuleSpec
from .matrix_state import MLSTM, GatedDelta, GatedDeltaSpec, MLSTMSpec
from .latent_attention import LatentAttention, LatentAttentionSpec, LatentNeed
from .moe import RoutedExperts, RoutedExpertsSpec
from .io import CappedHeadSpec, CappedLinearHead, LinearHead, ScaledHeadSpec, ScaledLinearHead, TokenEmbedding
