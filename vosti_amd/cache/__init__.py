from .manager import CacheError, CacheManager, OutOfPages
from .pool import CachePool

__all__ = ["CacheError", "CacheManager", "OutOfPages", "CachePool"]
