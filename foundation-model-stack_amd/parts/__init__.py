from . import attention, block, embedding, experts, feedforward, gated_delta, latent_attention, linear, norm, parallel, position, rglru  # noqa: F401  (register the parts)
from .attention import LayerCache, MultiHeadAttention
from .base import BranchOutput, FeedForward, Mixer, NormedRows, ParamSpec, Part, list_parts, make_part, part_attribute, register_part, unregister_part
from .block import PostNormBlock, PreNormBlock, ResidualStream, SandwichNormBlock
from .embedding import LinearHead, TokenEmbedding
from .experts import MLP, ExpertsFeedForward
from .feedforward import GatedLinearUnit
from .gated_delta import GatedDeltaRule
from .latent_attention import LatentAttention
from .linear import Linear
from .norm import ParameterizedNorm
from .parallel import ParallelMixers
from .rglru import RecurrentGatedUnit
from .position import PositionEncoding, RotaryEncoding, rope_frequencies
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

__all__ = [
    "LayerCache", "MultiHeadAttention", "Mixer", "FeedForward", "ParamSpec", "Part", "list_parts", "make_part", "part_attribute", "register_part",
    "unregister_part", "PreNormBlock", "ResidualStream", "LinearHead", "TokenEmbedding", "GatedLinearUnit", "Linear",
    "ParameterizedNorm", "PositionEncoding", "RotaryEncoding", "rope_frequencies", "LayerSpec", "ModelSpec",
    "PartSpec", "ScheduleEntry", "BranchOutput", "NormedRows", "SandwichNormBlock", "MLP", "ExpertsFeedForward", "LatentAttention", "GatedDeltaRule", "ParallelMixers",
]
