from .manager import CacheManager, OutOfPages, PagePool

__all__ = ["CacheManager", "OutOfPages", "PagePool"]
