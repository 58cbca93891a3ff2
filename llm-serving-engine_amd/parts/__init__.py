from .base import (
    BLOCKS,
    FEED_FORWARDS,
    LOGIT_PARTS,
    MIXERS,
    NORMS,
    PASS_PARTS,
    POSITIONS,
    CacheNeed,
    FixedState,
    PagedKeyValue,
    PagedNeed,
    SlotNeed,
    Part,
    Registry,
    STREAM_PARTS,
    TensorSpec,
)
from .norm import LayerNorm, LayerNormSpec, RMSNorm, RMSNormSpec
from .position import HeadLayout, NoPositionSpec, PositionEncoding, Rotary, RotarySpec, YarnScaling, rotary_frequencies
from .attention import Attention, AttentionSpec, Mixer
from .feed_forward import FeedForward, GatedMLP, GatedMLPSpec
from .block import Block, PreNormBlock, PreNormBlockSpec
from .model import DecoderModel, JoinedPass, JoinedPassSpec, LayerDefinition, LayerRun, ModelSpec, NamedPart
from .latent_attention import LatentAttention, LatentAttentionSpec
from .delta import GatedDelta, GatedDeltaSpec
from .experts import RoutedExperts, RoutedExpertsSpec

__all__ = [name for name in dir() if not name.startswith("_")]
