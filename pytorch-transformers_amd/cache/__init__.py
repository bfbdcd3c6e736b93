"""The cache: slots, pages, per-sequence state."""
from .paged import PAGE_SIZE, CacheError, CacheFull, PagedCache

__all__ = ["PAGE_SIZE", "CacheError", "CacheFull", "PagedCache"]
