"""Parts a model is put together from.  Importing the package registers the built-in kinds."""
from . import attention, block, feed_forward, norm, position  # noqa: F401  (registration)
from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, FusedRotation, PagedKVRequest, ParamDecl, Part,
                   StateRequest)
from .model import DecoderModel, build_model

__all__ = ["BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITIONS", "FusedRotation", "PagedKVRequest", "ParamDecl",
           "Part", "StateRequest", "DecoderModel", "build_model"]
