from .base import (
    BLOCKS,
    FEED_FORWARDS,
    LOGIT_PARTS,
    MIXERS,
    NORMS,
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
from .norm import RMSNorm, RMSNormSpec
from .position import HeadLayout, NoPositionSpec, PositionEncoding, Rotary, RotarySpec
from .attention import Attention, AttentionSpec, Mixer
from .feed_forward import FeedForward, GatedMLP, GatedMLPSpec
from .block import Block, PreNormBlock, PreNormBlockSpec
from .model import DecoderModel, LayerDefinition, LayerRun, ModelSpec, NamedPart

__all__ = [name for name in dir() if not name.startswith("_")]
