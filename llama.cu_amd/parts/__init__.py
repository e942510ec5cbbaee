"""Parts of a decoder and the registries that build them from specifications."""
from .base import (BuildContext, CacheNeed, LayerCache, ModelSpec, PagedKV, Part, PartSpec, RunEntry, ScaledRows, SlotState, TensorSpec, make_part,
                   register_part, registered_parts)
from . import norm, position, attention, ffn, block, model  # noqa: F401  (they register themselves)
from .model import DecoderModel

__all__ = ["BuildContext", "CacheNeed", "LayerCache", "ModelSpec", "PagedKV", "Part", "PartSpec", "RunEntry", "ScaledRows", "SlotState", "TensorSpec",
           "make_part", "register_part", "registered_parts", "DecoderModel"]
