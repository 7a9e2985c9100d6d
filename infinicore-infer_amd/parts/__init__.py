"""Parts a layer is put together from, and the layered model."""
from .base import (Block, CacheNeed, FeedForward, Mixer, Norm, Part, PositionEncoding, Runtime, build_part,
                   register_part, registered_parts)
from . import norm, rotary, attention, swiglu, block, embedding      # registers the built-in parts
from .model import DecoderModel, build_model

__all__ = ["Block", "CacheNeed", "FeedForward", "Mixer", "Norm", "Part", "PositionEncoding", "Runtime",
           "build_part", "register_part", "registered_parts", "DecoderModel", "build_model"]
