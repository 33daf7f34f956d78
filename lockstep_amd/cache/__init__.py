"""Cache manager: paged keys/values, block tables, state slots, prefix index."""

from .manager import (SUPPORTED_PAGE_SIZES, CacheAuditError, CacheGroup, CacheManager,
                      OutOfPages, PagePool)
from .prefix import PrefixIndex

__all__ = ["SUPPORTED_PAGE_SIZES", "CacheAuditError", "CacheGroup", "CacheManager",
           "OutOfPages", "PagePool", "PrefixIndex"]
