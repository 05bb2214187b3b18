from . import attention, block, embedding, feedforward, linear, norm, position  # noqa: F401  (register the parts)
from .attention import LayerCache, MultiHeadAttention
from .base import BranchOutput, FeedForward, Mixer, NormedRows, ParamSpec, Part, list_parts, make_part, part_attribute, register_part, unregister_part
from .block import PreNormBlock, ResidualStream
from .embedding import LinearHead, TokenEmbedding
from .feedforward import GatedLinearUnit
from .linear import Linear
from .norm import ParameterizedNorm
from .position import PositionEncoding, RotaryEncoding, rope_frequencies
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

__all__ = [
    "LayerCache", "MultiHeadAttention", "Mixer", "FeedForward", "ParamSpec", "Part", "list_parts", "make_part", "part_attribute", "register_part",
    "unregister_part", "PreNormBlock", "ResidualStream", "LinearHead", "TokenEmbedding", "GatedLinearUnit", "Linear",
    "ParameterizedNorm", "PositionEncoding", "RotaryEncoding", "rope_frequencies", "LayerSpec", "ModelSpec",
    "PartSpec", "ScheduleEntry", "BranchOutput", "NormedRows",
]
