"""The parts a layer is put together from, and the registries of their kinds."""
from .base import (Block, CacheSpec, FeedForward, Mixer, Norm, Part, PositionEncoding, StateSpec, WeightSpec,
                   make_part, register_block, register_feed_forward, register_mixer, register_norm,
                   register_position, registered_kinds)
from .attention import (DifferentialAttention, GatedTiedValueAttention, LatentAttention, PagedAttention,
                        RotaryLatentAttention, TiedValueAttention)
from .block import DepthAverage, PreNormBlock, SandwichBlock, SideBySideBlock
from .loop import LoopEntry, NoMixer
from .embedding import OutputHead, TokenEmbedding
from .experts import RoutedExperts
from .feed_forward import DenseFeedForward, SwiGLU
from .linear import linear
from .norm import RMSNorm
from .parallel import ParallelMixer
from .position import NoPosition, RotaryEncoding
from .recurrent import GatedDeltaRule, GatedLinearRecurrence, LightningAttention, MinGRU, StateSpaceDuality
from .streams import BigramEmbedding, StreamBlock, StreamsNorm, StreamUpdate

__all__ = ["Block", "CacheSpec", "FeedForward", "Mixer", "Norm", "Part", "PositionEncoding", "StateSpec",
           "WeightSpec", "make_part", "register_block", "register_feed_forward", "register_mixer", "register_norm",
           "register_position", "registered_kinds", "PagedAttention", "PreNormBlock", "OutputHead",
           "TokenEmbedding", "SwiGLU", "linear", "RMSNorm", "NoPosition", "RotaryEncoding", "TiedValueAttention",
           "SandwichBlock", "RoutedExperts", "ParallelMixer", "GatedDeltaRule", "LatentAttention", "SideBySideBlock",
           "LoopEntry", "NoMixer", "StateSpaceDuality", "DifferentialAttention", "MinGRU", "DepthAverage",
           "GatedTiedValueAttention", "RotaryLatentAttention", "DenseFeedForward", "GatedLinearRecurrence",
           "LightningAttention", "BigramEmbedding", "StreamBlock", "StreamsNorm", "StreamUpdate"]
