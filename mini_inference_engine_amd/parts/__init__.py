from .attention import Attention
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, Block, CacheBinding, CacheRequirement, DecoderSpec,
                   FeedForward, FixedState, LayerCall, Mixer, Norm, PagedKV, ParamSpec, Part, PositionEncoding,
                   Source, WEIGHT_TRANSFORMS, register_block, register_feed_forward, register_mixer, register_norm,
                   register_position_encoding, register_weight_transform)
from .block import BranchNormBlock, PreNormBlock
from .embedding import Embedding, LMHead
from .latent_attention import LatentAttention, PagedLatent
from .rglru import RGLRU, RecurrentState
from .rmsnorm import RMSNorm
from .rope import NoPosition, RotaryHalfSplit, RotaryInterleaved, rotary_tables
from .routed_experts import RoutedExperts
from .swiglu import SwiGLU
