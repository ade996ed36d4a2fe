"""Parts of a decoder and the registries that build them from specifications."""
from .base import (BuildContext, CacheNeed, LayerCache, ModelSpec, NormedRows, PagedKV, Part, PartSpec, RunEntry, ScaledRows, SeveralNeeds, SlotState,
                   TensorSpec, make_part,
                   register_part, registered_parts)
from . import norm, position, attention, latent, delta, retention, rglru, selective_scan, side_by_side, ffn, moe, block, model  # noqa: F401  (they register themselves)
from .model import DecoderModel

__all__ = ["BuildContext", "CacheNeed", "LayerCache", "ModelSpec", "NormedRows", "PagedKV", "Part", "PartSpec", "RunEntry", "ScaledRows", "SeveralNeeds", "SlotState", "TensorSpec",
           "make_part", "register_part", "registered_parts", "DecoderModel"]
