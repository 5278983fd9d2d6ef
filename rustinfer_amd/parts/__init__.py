from .base import (FeedForward, Mixer, Norm, PagedKVNeed, ParamSpec, Part, PositionEncoding,
                   ProjectedPart, ProjectionSet, Runtime, StateNeed, CompoundNeed, stored_to)
from .norm import LayerNorm, OutputRMSNorm, RMSNorm
from .rope import RotaryEmbedding, rotary_frequencies
from .linear import Linear
from .embed import Embedding, LMHead
from .mlp import DenseMLP, MoEFeedForward, PolyNormMLP, SwiGLUMLP
from .attention import LatentAttention, PagedAttention, WindowAttention
from .recurrent import (ChannelGatedDeltaRule, GatedDeltaRule, GatedLinearAttention, GeneralDeltaRule, LightningAttention,
                        Retention, StateSpaceMixer)
from .block import Hidden, ParallelBlock, PostNormBlock, PreNormBlock, SandwichBlock, TokenShift, TwoMixers
from .registry import (MIXERS, FEED_FORWARDS, NORMS, POSITION_ENCODINGS, register_mixer,
                       register_feed_forward, register_norm, register_position_encoding,
                       make_part)

register_mixer("two_mixers", TwoMixers)
