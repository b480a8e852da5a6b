from .base import (CATEGORIES, KernelSet, Norm, NormedDelta, PagedKV, Part, Runtime, SlotState, StreamSums, UnnormedRows, build_part,
                   register_part, registered)
from . import (norm, position, linear, feed_forward, attention, block, embedding, latent_attention,  # noqa: F401
               selective_scan, routed_experts, gated_attention, retention, parallel, rglru,      # (registers the kinds)
               differential_attention, delta_rule)
from .attention import Attention
from .block import NoFeedForward, PreNormBlock, SandwichBlock, ScaledPreNormBlock
from .delta_rule import GatedDeltaRule
from .differential_attention import DifferentialAttention
from .gated_attention import GatedAttention
from .parallel import ParallelMixers
from .retention import Retention
from .rglru import RecurrentGatedUnit
from .embedding import Embedding, LinearHead, PairHashEmbedding
from .feed_forward import SwiGLU
from .latent_attention import LatentAttention
from .routed_experts import RoutedExperts
from .selective_scan import SelectiveScan
from .linear import Linear
from .norm import RMSNorm
from .position import NoPosition, RotaryHalf

__all__ = ["CATEGORIES", "KernelSet", "Norm", "PagedKV", "Part", "Runtime", "SlotState", "StreamSums", "UnnormedRows",
           "build_part", "register_part", "registered",
           "NormedDelta", "GatedAttention", "DifferentialAttention", "GatedDeltaRule", "ParallelMixers", "Retention", "RecurrentGatedUnit", "ScaledPreNormBlock",
           "LatentAttention", "RoutedExperts", "SelectiveScan", "SandwichBlock", "NoFeedForward",
           "PairHashEmbedding", "Attention", "PreNormBlock", "Embedding", "LinearHead", "SwiGLU", "Linear", "RMSNorm", "NoPosition",
           "RotaryHalf"]
