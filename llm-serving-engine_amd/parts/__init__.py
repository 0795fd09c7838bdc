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
from .position import HeadLayout, LinearScaling, NoPositionSpec, PositionEncoding, Rotary, RotarySpec, WavelengthScaling, YarnScaling, rotary_frequencies
from .attention import Attention, AttentionSpec, Mixer
from .feed_forward import FeedForward, GatedMLP, GatedMLPSpec
from .block import Block, OutputNormBlock, OutputNormBlockSpec, PendingNormed, PreNormBlock, PreNormBlockSpec, SandwichBlock, SandwichBlockSpec
from .model import AddedPass, AddedPassSpec, DecoderModel, JoinedPass, JoinedPassSpec, LayerDefinition, LayerRun, ModelSpec, NamedPart, SoftCap, SoftCapSpec
from .latent_attention import LatentAttention, LatentAttentionSpec
from .delta import GatedDelta, GatedDeltaSpec
from .experts import RoutedExperts, RoutedExpertsSpec
from .normed_attention import NormedAttention, NormedAttentionSpec
from .decay_attention import DecayAttention, DecayAttentionSpec
from .hyper import HyperBlock, HyperBlockSpec, PendingWrite, StreamCopies, StreamCopiesSpec, StreamNorm, StreamNormSpec
from .recurrent import GatedRecurrence, GatedRecurrenceSpec
from .parallel import ParallelMixers, ParallelMixersSpec

__all__ = [name for name in dir() if not name.startswith("_")]
