from .base import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITIONS, BuildContext, EntryMeta, PagedCacheView, Part,
                   Registry, ResidualStream, StateView, StepContext, Workspace)
from . import attention, block, embedding, mlp, norm, rope  # noqa: F401  (registers the built-in parts)

__all__ = ["BLOCKS", "FEED_FORWARDS", "MIXERS", "NORMS", "POSITIONS", "BuildContext", "EntryMeta", "PagedCacheView",
           "Part", "Registry", "ResidualStream", "StateView", "StepContext", "Workspace"]
