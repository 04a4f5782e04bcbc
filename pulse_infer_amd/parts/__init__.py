from .base import (BLOCKS, EMBEDDINGS, FEED_FORWARDS, HEADS, MIXERS, NORMS, POSITIONS, BuildContext, EntryMeta,
                   PagedCacheView, Part, Registry, ResidualStream, StateView, StepContext, Workspace)
from . import attention, block, embedding, mlp, norm, rope  # noqa: F401  (registers the built-in parts)

__all__ = ["BLOCKS", "EMBEDDINGS", "FEED_FORWARDS", "HEADS", "MIXERS", "NORMS", "POSITIONS", "BuildContext", "EntryMeta",
           "PagedCacheView", "Part", "Registry", "ResidualStream", "StateView", "StepContext", "Workspace"]
