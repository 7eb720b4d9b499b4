"""Slot-per-sequence paged key/value cache and per-sequence state."""
from .pages import PAGE_TOKENS, CacheError, CacheFull, FreeList, GroupPages, SlotBook, blocks_for
