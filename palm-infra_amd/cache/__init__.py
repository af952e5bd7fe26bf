"""Slots, pages, key/value groups and per-sequence state."""
from .pool import PAGE_TOKENS, CacheFull, CacheMisuse, FreeList, PageTable, pages_for
from .cache import (KVGroup, KVNeed, LayerCache, ModelCache, PagedGroup, RowsGroup, RowsNeed, RowsView, StateGroup,
                    StateNeed)

__all__ = ["PAGE_TOKENS", "CacheFull", "CacheMisuse", "FreeList", "PageTable", "pages_for", "KVGroup", "KVNeed",
           "LayerCache", "ModelCache", "PagedGroup", "RowsGroup", "RowsNeed", "RowsView", "StateGroup", "StateNeed"]
