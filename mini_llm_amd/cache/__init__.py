from .manager import NO_PAGE, CacheError, CacheManager, RequestCache
from .pages import OutOfPages, PagePool, blocks_for, first_needed_block

__all__ = ["NO_PAGE", "CacheError", "CacheManager", "RequestCache", "OutOfPages", "PagePool", "blocks_for", "first_needed_block"]
