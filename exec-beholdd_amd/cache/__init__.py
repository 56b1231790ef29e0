"""Per-sequence storage between steps: slots, paged keys and values, fixed-size state."""

from .sequence_cache import CacheError, CacheFull, CachePlan, SequenceCache

__all__ = ["CacheError", "CacheFull", "CachePlan", "SequenceCache"]
